"""The cache manager: which pages and which state slot each request holds.

Host-side books only; the memory itself is in cache/storage.py. The reference's
cache is private to one context (a table of 64-token blocks per layer, allocated
lazily by ``kv_reserve``, src/model.c:309-330, and freed only with the context,
src/model.c:217-230). Here pages come from shared pools:

* Schedule entries whose mixers ask for paged storage are put into **groups** by what
  they ask for (row widths and window). A group has its own page ids, its own pool and,
  per request, its own block table; all entries of a group use the same page id for the
  same tokens, each in its own memory.
* A request's block ``b`` of a group covers positions ``b * page_tokens ..``; the table
  is indexed by absolute block number.
* Pages go back to the pool when the request is released, and, in a group with a
  window ``W``, as soon as every position on the page is ``<= next_pos - W`` for the
  request's next position: no later query can see them.
* ``fork`` gives a new request the cache of another (src/model.c:271-301): whole pages are
  shared and counted, the last, partly filled page is copied, because both will write there.
  A shared page is never written: a request writes only at and beyond its own length.
* Every request also holds one **state slot** (an index below ``n_slots``) from
  admission to release, for parts that keep per-request state of fixed size; the
  device block tables are indexed by it as well.
"""
from dataclasses import dataclass, field

import numpy as np

from ..parts.base import FixedState, PagedKV
from ..status import EINVAL, ENOMEM, ENOTSUP, ERANGE, EngineError, fail
from .pages import OutOfPages, PagePool


@dataclass
class Group:
    index: int
    k_width: int
    v_width: int
    window: int
    entries: list = field(default_factory=list)     # schedule entries that store here


@dataclass
class Held:
    """What one request holds."""
    req_id: object
    slot: int
    length: int = 0                                  # tokens whose cache rows are valid
    tables: list = field(default_factory=list)       # per group: page id per absolute block, -1 = gone
    reserved: int = 0                                # tokens beyond `length` that have pages


class CacheManager:
    def __init__(self, needs, page_tokens, n_pages, n_slots, max_context):
        """``needs[i]`` is schedule entry ``i``'s PagedKV, FixedState or None.
        ``n_pages`` is the size of every group's pool."""
        if page_tokens <= 0 or n_slots <= 0 or max_context <= 0:
            fail(EINVAL, "cache manager: page_tokens, n_slots and max_context must be positive")
        self.page_tokens = page_tokens
        self.max_context = max_context
        self.max_blocks = -(-max_context // page_tokens)
        self.n_slots = n_slots
        self.groups = []
        self.entry_group = []            # per schedule entry: group index or None
        self.state_entries = {}          # schedule entry -> n_floats
        by_key = {}
        for i, need in enumerate(needs):
            if isinstance(need, PagedKV):
                key = (need.k_width, need.v_width, need.window)
                if key not in by_key:
                    by_key[key] = len(self.groups)
                    self.groups.append(Group(len(self.groups), *key))
                self.groups[by_key[key]].entries.append(i)
                self.entry_group.append(by_key[key])
            else:
                self.entry_group.append(None)
                if isinstance(need, FixedState):
                    self.state_entries[i] = need.n_floats
        self.pools = [PagePool(n_pages) for _ in self.groups]
        self._free_slots = list(range(n_slots - 1, -1, -1))
        self.held = {}
        self.appended = [[] for _ in self.groups]    # per group: (slot, block, page) since last drain

    # ---- admission and release ------------------------------------------
    def admit(self, req_id):
        if req_id in self.held:
            fail(EINVAL, f"request {req_id!r} is already admitted")
        if not self._free_slots:
            raise EngineError(ENOMEM, f"no state slot is free ({self.n_slots} in use)")
        h = Held(req_id, self._free_slots.pop(), tables=[[] for _ in self.groups])
        self.held[req_id] = h
        return h

    def release(self, req_id):
        h = self.held.pop(req_id, None)
        if h is None:
            fail(EINVAL, f"request {req_id!r} is released but not admitted")
        for g, table in enumerate(h.tables):
            self.pools[g].give_back([p for p in table if p >= 0])
            # Entries not yet sent to the device name a slot that the next request may take before
            # the next drain: two entries for one (slot, block) in one scatter have no order.
            self.appended[g] = [a for a in self.appended[g] if a[0] != h.slot]
        self._free_slots.append(h.slot)

    def fork(self, src_id, new_id):
        """Admits ``new_id`` with the cache contents of ``src_id``: the same length, the whole
        pages shared, a page of its own for the last, partly filled block. All or nothing.
        Returns what the caller has to copy in device memory before either request runs again:
        ``(page_copies, slot_copy)`` with page_copies = [(group, from_page, to_page)] and
        slot_copy = (from_slot, to_slot)."""
        src = self.held.get(src_id)
        if src is None:
            fail(EINVAL, f"request {src_id!r} is forked but not admitted")
        if new_id in self.held:
            fail(EINVAL, f"request {new_id!r} is already admitted")
        if src.reserved:
            fail(EINVAL, f"request {src_id!r} is forked in the middle of a step")
        if not self._free_slots:
            raise EngineError(ENOMEM, f"no state slot is free ({self.n_slots} in use)")
        P = self.page_tokens
        full, partial = src.length // P, src.length % P != 0
        if partial:
            for g, pool in enumerate(self.pools):
                if pool.n_free < 1:
                    raise OutOfPages(f"fork of {src_id!r}: group {g} has no page for the last block")
        h = Held(new_id, self._free_slots.pop(), length=src.length, tables=[])
        copies = []
        for g, pool in enumerate(self.pools):
            table = list(src.tables[g][:full])
            pool.share([p for p in table if p >= 0])
            if partial:
                own = pool.take(1)[0]
                copies.append((g, src.tables[g][full], own))
                table.append(own)
            for b, page in enumerate(table):
                if page >= 0:
                    self.appended[g].append((h.slot, b, page))
            h.tables.append(table)
        self.held[new_id] = h
        return copies, (src.slot, h.slot)

    # ---- pages ---------------------------------------------------------------
    def _first_needed_block(self, group, next_pos):
        """Blocks before this one hold only keys that no query at ``next_pos`` or later sees."""
        if group.window <= 0:
            return 0
        return max(0, next_pos - group.window + 1) // self.page_tokens

    def pages_needed(self, req_id, n_new):
        """Per group, the pages ``reserve(req_id, n_new)`` would take (the request may be
        one that is not admitted yet)."""
        h = self.held.get(req_id)
        length = h.length if h else 0
        last_block = (length + n_new - 1) // self.page_tokens
        out = []
        for g in self.groups:
            have = len(h.tables[g.index]) if h else 0
            out.append(max(0, last_block + 1 - have))
        return out

    def can_reserve(self, wanted):
        """Whether the pools can serve all of ``wanted`` = [(req_id, n_new), ...] together."""
        total = [0] * len(self.groups)
        for req_id, n_new in wanted:
            for g, n in enumerate(self.pages_needed(req_id, n_new)):
                total[g] += n
        return all(total[g] <= self.pools[g].n_free for g in range(len(self.groups)))

    def reserve(self, req_id, n_new):
        """Pages for positions ``length .. length + n_new - 1`` in every group, all or
        nothing. Raises OutOfPages (nothing taken) or ERANGE past ``max_context``."""
        h = self.held[req_id]
        if n_new <= 0:
            fail(EINVAL, f"request {req_id!r}: a step needs at least one token")
        if h.length + n_new > self.max_context:
            raise EngineError(ERANGE, f"request {req_id!r}: {h.length} + {n_new} tokens exceed the "
                                      f"context limit {self.max_context}")        # src/model.c:558
        need = self.pages_needed(req_id, n_new)
        for g, n in enumerate(need):
            if n > self.pools[g].n_free:
                raise OutOfPages(f"request {req_id!r}: group {g} needs {n} pages, "
                                 f"{self.pools[g].n_free} of {self.pools[g].n_pages} free")
        for g, n in enumerate(need):
            table = h.tables[g]
            for page in self.pools[g].take(n):
                self.appended[g].append((h.slot, len(table), page))
                table.append(page)
        h.reserved = max(h.reserved, n_new)

    def rollback(self, req_id):
        """Gives back pages that lie wholly beyond the committed length (after a step that
        was reserved for but did not run)."""
        h = self.held[req_id]
        keep = -(-h.length // self.page_tokens)
        for g, table in enumerate(h.tables):
            extra = [p for p in table[keep:] if p >= 0]
            del table[keep:]
            self.pools[g].give_back(extra)
            self.appended[g] = [a for a in self.appended[g] if not (a[0] == h.slot and a[1] >= keep)]
        h.reserved = 0

    def commit(self, req_id, n_new):
        """The step ran: ``n_new`` more tokens are valid. Pages a window has passed go back."""
        h = self.held[req_id]
        if n_new > h.reserved:
            fail(EINVAL, f"request {req_id!r}: {n_new} tokens committed, {h.reserved} reserved")
        h.length += n_new
        h.reserved = 0
        for g in self.groups:
            if g.window > 0:
                table = h.tables[g.index]
                stop = min(self._first_needed_block(g, h.length), len(table))
                gone = [table[b] for b in range(stop) if table[b] >= 0]
                if gone:
                    for b in range(stop):
                        table[b] = -1
                    self.pools[g.index].give_back(gone)

    def truncate(self, req_id, length):
        """Lowers the valid length (src/model.c:305) and gives back pages wholly beyond it.
        Refused if a window group has already let go of pages the shorter sequence needs."""
        h = self.held[req_id]
        if not 0 <= length <= h.length:
            fail(EINVAL, f"request {req_id!r}: cannot truncate {h.length} tokens to {length}")
        for g in self.groups:
            first = self._first_needed_block(g, length)
            if any(p < 0 for p in h.tables[g.index][first:-(-length // self.page_tokens)]):
                fail(ENOTSUP, f"request {req_id!r}: the window has released pages before {length}")
        if length % self.page_tokens:
            for g, pool in enumerate(self.pools):
                page = h.tables[g][length // self.page_tokens]
                if page >= 0 and pool.holders(page) > 1:
                    fail(ENOTSUP, f"request {req_id!r}: position {length} lies on a page shared with a fork")
        h.length = length
        self.rollback(req_id)

    # ---- what a step needs to know ---------------------------------------------
    def slot_rows(self, req_id, group, start, count):
        """Cache row (page * page_tokens + offset) of positions start .. start + count - 1."""
        table = self.held[req_id].tables[group]
        P = self.page_tokens
        first, last = start // P, (start + count - 1) // P
        pages = np.asarray(table[first:last + 1], dtype=np.int64)
        assert count <= 0 or (len(pages) == last + 1 - first and pages.min() >= 0), \
            "a position about to be written has no page"
        pos = np.arange(start, start + count, dtype=np.int64)
        return (pages[pos // P - first] * P + pos % P).astype(np.int32)

    def drain_appended(self, group):
        """(slot, block, page) entries added to block tables since the last call."""
        out, self.appended[group] = self.appended[group], []
        if len({(a[0], a[1]) for a in out}) != len(out):       # the last entry of a (slot, block) is the one that holds
            out = list({(a[0], a[1]): a for a in out}.values())
        return out

    # ---- accounting ----------------------------------------------------------
    def stats(self):
        return {"groups": [{"window": g.window, "entries": len(g.entries), "pages": p.n_pages,
                            "held": p.n_held, "high_water": p.high_water, "reused": p.reused}
                           for g, p in zip(self.groups, self.pools)],
                "slots_held": self.n_slots - len(self._free_slots), "requests": len(self.held)}

    def check(self):
        """Raises AssertionError unless every page is either free or held by exactly as many
        requests as the pool counts for it (one, unless forks share it), no page beyond a
        request's last whole block is shared, and every slot is free or held once."""
        for g, pool in enumerate(self.pools):
            pool.check()
            count = {}
            for h in self.held.values():
                own = [p for p in h.tables[g] if p >= 0]
                assert len(own) == len(set(own)), f"group {g}: request {h.req_id!r} holds a page twice"
                for p in own:
                    count[p] = count.get(p, 0) + 1
                for p in h.tables[g][h.length // self.page_tokens:]:
                    assert p < 0 or pool.holders(p) == 1, f"group {g}: a page that will be written is shared"
            assert len(count) == pool.n_held, f"group {g}: {pool.n_held} pages out, {len(count)} in tables"
            for p, n in count.items():
                assert pool.holders(p) == n, f"group {g}: page {p} has {pool.holders(p)} holders, {n} tables name it"
        slots = [h.slot for h in self.held.values()]
        assert len(slots) == len(set(slots)), "a state slot is held twice"
        assert sorted(slots + self._free_slots) == list(range(self.n_slots)), "a state slot is lost"


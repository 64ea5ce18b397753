"""The step function: one batch of (request, its next tokens) through the model.

``Engine.step`` runs only the tokens it is given, from the cache earlier steps
left, and returns the logits at the wanted places. It is what generation, the
command line and trace replay all drive; there is no other forward pass.
Reference: ``forward_impl`` (src/model.c:545-640) with its two batch shapes
(src/model.c:642-650) made one.
"""
import numpy as np
import torch

from ..cache import CacheManager, CacheStorage, OutOfPages
from ..status import EINVAL, fail
from .batch import Entry, GroupInputs, IntStaging, StepInputs, as_i32


class Engine:
    def __init__(self, model, ops, page_tokens=16, n_pages=None, max_tokens=None, max_seqs=8,
                 max_context=None):
        """``n_pages`` pages per group, or ``max_tokens`` (the most tokens live requests
        hold at once, each request's count rounded up to whole pages) from which it follows.
        ``max_context`` bounds one request's length (default: what the pool can hold)."""
        if n_pages is None:
            if max_tokens is None:
                fail(EINVAL, "engine: give n_pages or max_tokens")
            n_pages = -(-int(max_tokens) // page_tokens)
        if max_context is None:
            max_context = n_pages * page_tokens
        self.model, self.ops = model, ops
        self.manager = CacheManager(model.cache_needs(), page_tokens, n_pages, max_seqs, max_context)
        self.storage = CacheStorage(self.manager, model.dtype, ops.device)
        self.staging = IntStaging(ops.device)
        self.vocab_size = model.vocab_size
        self.steps_run = 0

    # ---- requests ------------------------------------------------------------
    def has(self, req_id):
        return req_id in self.manager.held

    def length(self, req_id):
        return self.manager.held[req_id].length

    def release(self, req_id):
        """The request is finished: its pages and its slot are given back."""
        self.manager.release(req_id)

    # ---- one step ------------------------------------------------------------
    def step(self, entries):
        """``entries``: a list of Entry or (req_id, tokens, want). A request seen for the
        first time is admitted. Returns fp32 logits [R, vocab] on the device, rows in the
        order of the entries and of each entry's ``want``; the tensor is a view of a work
        buffer and is overwritten by the next step. On an error nothing is kept: lengths,
        pages and admissions are as before the call."""
        entries = [e if isinstance(e, Entry) else Entry(*e) for e in entries]
        if not entries:
            fail(EINVAL, "step: no entries")
        seen = set()
        for e in entries:
            if e.req_id in seen:
                fail(EINVAL, f"step: request {e.req_id!r} appears twice")
            seen.add(e.req_id)
            if len(e.tokens) == 0:
                fail(EINVAL, f"step: request {e.req_id!r} brings no tokens")       # src/model.c:555
            for t in e.tokens:
                if not 0 <= int(t) < self.vocab_size:
                    fail(EINVAL, f"step: token id {t} of request {e.req_id!r} is outside the "
                                 f"vocabulary of {self.vocab_size}")                # src/model.c:568
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    fail(EINVAL, f"step: request {e.req_id!r} wants logits at place {w} of {len(e.tokens)} tokens")
        mgr = self.manager
        admitted, reserved = [], []
        try:
            for e in entries:
                if e.req_id not in mgr.held:
                    h = mgr.admit(e.req_id)
                    admitted.append(e.req_id)
                    self.storage.clear_slot(h.slot)
                mgr.reserve(e.req_id, len(e.tokens))
                reserved.append(e.req_id)
            step = self._inputs(entries)
            logits = self.ops.scratch("logits", (max(step.n_logit_rows, 1), self.vocab_size), torch.float32)
            logits = logits[:step.n_logit_rows]
            self.model.forward(self.ops, step, self.storage.views, logits)
        except BaseException:
            for r in reserved:
                mgr.rollback(r)
            for r in admitted:
                mgr.release(r)
            raise
        for e in entries:
            mgr.commit(e.req_id, len(e.tokens))
        self.steps_run += 1
        return logits

    def _inputs(self, entries):
        mgr = self.manager
        T = sum(len(e.tokens) for e in entries)
        S = len(entries)
        tokens = np.empty(T, np.int32)
        positions = np.empty(T, np.int32)
        token_slot = np.empty(T, np.int32)
        q_start = np.zeros(S + 1, np.int32)
        seq_slot = np.empty(S, np.int32)
        seq_len = np.empty(S, np.int32)
        rows = []
        slot_maps = [np.empty(T, np.int32) for _ in mgr.groups]
        at = 0
        max_q = max_len = 0
        for s, e in enumerate(entries):
            h = mgr.held[e.req_id]
            n = len(e.tokens)
            tokens[at:at + n] = e.tokens
            positions[at:at + n] = np.arange(h.length, h.length + n, dtype=np.int32)
            token_slot[at:at + n] = h.slot
            q_start[s + 1] = at + n
            seq_slot[s] = h.slot
            seq_len[s] = h.length + n
            rows.extend(at + int(w) for w in e.want)
            for g in range(len(mgr.groups)):
                slot_maps[g][at:at + n] = mgr.slot_rows(e.req_id, g, h.length, n)
            max_q = max(max_q, n)
            max_len = max(max_len, h.length + n)
            at += n
        arrays = [tokens, positions, token_slot, q_start, seq_slot, seq_len, as_i32(rows)]
        dirty = []
        for g in range(len(mgr.groups)):
            app = mgr.drain_appended(g)
            dirty.append(len(app))
            arrays.append(slot_maps[g])
            arrays.append(as_i32([slot * mgr.max_blocks + block for slot, block, _ in app]))
            arrays.append(as_i32([page for _, _, page in app]))
        views = self.staging.upload(arrays)
        step = StepInputs(T, S, len(rows))
        (step.tokens, step.positions, step.token_slot, step.q_start, step.seq_slot, step.seq_len,
         step.logit_rows) = views[:7]
        step.max_q_len, step.max_seq_len = max_q, max_len
        step.host = dict(tokens=tokens, positions=positions, token_slot=token_slot, q_start=q_start,
                         seq_slot=seq_slot, seq_len=seq_len, logit_rows=as_i32(rows))
        for g in range(len(mgr.groups)):
            slot_map, idx, val = views[7 + 3 * g:10 + 3 * g]
            table = self.storage.block_tables[g]
            if dirty[g]:
                self.ops.scatter_i32(table.view(-1), idx, val)
            step.groups.append(GroupInputs(table, slot_map))
        return step

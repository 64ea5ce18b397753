"""The step function: one batch of (request, its next tokens) through the model.

``Engine.step`` runs only the tokens it is given, from the cache earlier steps
left, and returns the logits at the wanted places. It is what generation, the
command line and trace replay all drive; there is no other forward pass.
Reference: ``forward_impl`` (src/model.c:545-640) with its two batch shapes
(src/model.c:642-650) made one.
"""
import numpy as np
import torch

from .. import memory
from ..cache import CacheManager, CacheStorage
from ..status import EINVAL, ENOTSUP, fail
from .batch import Entry, GroupInputs, IntStaging, StepInputs, as_i32


class Engine:
    GRAPH_MAX_TOKENS = 256        # decode-only steps up to this many requests replay a captured graph
    GRAPH_LEN_BUCKET = 256        # a graph serves request lengths up to a multiple of this
    BATCH_BUCKET = 8              # decode steps of more requests than this are filled up to a multiple of it
    GRAPHS_KEPT = 96              # graphs held at a time; the one replayed longest ago goes first

    def __init__(self, model, ops, page_tokens=16, n_pages=None, max_tokens=None, max_seqs=8,
                 max_context=None, graphs=True):
        """``n_pages`` pages per group, or ``max_tokens`` (the most tokens live requests
        hold at once, each request's count rounded up to whole pages) from which it follows.
        ``max_context`` bounds one request's length (default: what the pool can hold).
        ``graphs``: steps in which every request brings one token (decode) are captured
        into a HIP graph per (batch size, length bucket) the second time their shape is seen
        and replayed from then on; the integers of a step still travel before the replay."""
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
        self._short_rows = int(getattr(model, "short_request_rows", 0))      # see _inputs
        self.steps_run = 0
        self.use_graphs = bool(graphs) and bool(getattr(model, "graph_safe", False))
        self._graphs = {}
        self._graph_seen = set()
        self.graph_replays = 0
        self.profile = None           # while timing: {"prefill" | "decode": {part: milliseconds}}

    # ---- requests ------------------------------------------------------------
    def has(self, req_id):
        return req_id in self.manager.held

    def length(self, req_id):
        return self.manager.held[req_id].length

    def release(self, req_id):
        """The request is finished: its pages and its slot are given back."""
        self.manager.release(req_id)

    def truncate(self, req_id, length):
        """Cuts the request back to its first ``length`` tokens (src/model.c:305): the next step's tokens
        follow position ``length - 1``. Pages wholly beyond go back to the pool; rows beyond ``length`` on
        the last page stay and are overwritten. Refused (ENOTSUP), with nothing changed, if the model
        keeps per-request state of fixed size (it cannot be wound back), if a window has already given
        back pages that the shorter sequence would see, or if the cut falls on a page shared with a fork."""
        if req_id not in self.manager.held:
            fail(EINVAL, f"request {req_id!r} is truncated but not admitted")
        if self.manager.state_entries and length < self.manager.held[req_id].length:
            fail(ENOTSUP, f"request {req_id!r}: a model with per-request state of fixed size cannot be cut back")
        self.manager.truncate(req_id, int(length))

    def fork(self, src_id, new_id):
        """Admits ``new_id`` holding what ``src_id`` holds (src/model.c:271-301): whole pages are
        shared, the last, partly filled page and the state slot are copied. Both requests go on
        independently afterwards. On an error (no page, no slot) nothing is taken."""
        copies, (from_slot, to_slot) = self.manager.fork(src_id, new_id)
        P = self.manager.page_tokens
        for group, src, dst in copies:
            for e in self.manager.groups[group].entries:
                view = self.storage.views[e]
                view.k[dst * P:(dst + 1) * P].copy_(view.k[src * P:(src + 1) * P])
                view.v[dst * P:(dst + 1) * P].copy_(view.v[src * P:(src + 1) * P])    # a page's block, whatever its inner order
        for e in self.manager.state_entries:
            state = self.storage.views[e].state
            state[to_slot].copy_(state[from_slot])

    # ---- timing by part (src/model.h:75-79; reported by --profile, src/ops.c:593-603) ----
    def profile_start(self):
        """From now on every step's device time is booked by part (embed, qkv, attn, wo, gate_up,
        silu, down, head; the rest, norms, rotary, cache stores and partial sums, as glue),
        under ``prefill`` if the step holds a prompt portion, else under ``decode``. Steps run
        eagerly and the host waits for each, so the total is larger than without timing."""
        self.ops.timing(True)
        self.profile = {"prefill": {}, "decode": {}}

    def profile_stop(self):
        out, self.profile = self.profile, None
        self.ops.timing(False)
        return out

    def _book_times(self, stage):
        times = self.ops.take_times()
        book = self.profile[stage]
        named = sum(v for k, v in times.items() if k != "total")
        times["glue"] = max(times.pop("total", 0.0) - named, 0.0)
        for k, v in times.items():
            book[k] = book.get(k, 0.0) + v

    # ---- one step ------------------------------------------------------------
    def step(self, entries, fed=None):
        """``entries``: a list of Entry or (req_id, tokens, want). A request seen for the
        first time is admitted. Returns fp32 logits [R, vocab] on the device, rows in the
        order of the entries and of each entry's ``want``; the tensor is a view of a work
        buffer and is overwritten by the next step. On an error nothing is kept: lengths,
        pages and admissions are as before the call.

        ``fed``: ``(source, {entry index: row})``: the single token of each of these entries is
        ``source[row]``, an int32 tensor on the device (what the sampler chose after the step before,
        not yet read by the host); the token the entry itself names is ignored. The host can then
        enqueue a step before it knows the tokens of the one before."""
        entries = [e if isinstance(e, Entry) else Entry(*e) for e in entries]
        if not entries:
            fail(EINVAL, "step: no entries")
        fed_rows = {} if fed is None else dict(fed[1])
        for i in fed_rows:
            if not 0 <= i < len(entries) or len(entries[i].tokens) != 1:
                fail(EINVAL, "step: a token taken from the device belongs to an entry with exactly one token")
            entries[i] = Entry(entries[i].req_id, [0], entries[i].want)
        if fed_rows and (fed[0].dtype != torch.int32 or not fed[0].is_contiguous()
                         or not all(0 <= r < fed[0].numel() for r in fed_rows.values())):
            fail(EINVAL, "step: tokens taken from the device come from a contiguous int32 tensor that holds their rows")
        if self._is_plain_decode(entries):
            return self._decode_step(entries, fed, fed_rows)
        seen = set()
        for e in entries:
            if e.req_id in seen:
                fail(EINVAL, f"step: request {e.req_id!r} appears twice")
            seen.add(e.req_id)
            n = len(e.tokens)
            if n == 0:
                fail(EINVAL, f"step: request {e.req_id!r} brings no tokens")       # src/model.c:555
            toks = np.asarray(e.tokens, dtype=np.int64)
            if toks.min() < 0 or toks.max() >= self.vocab_size:
                bad = int(toks[(toks < 0) | (toks >= self.vocab_size)][0])
                fail(EINVAL, f"step: token id {bad} of request {e.req_id!r} is outside the "
                             f"vocabulary of {self.vocab_size}")                    # src/model.c:568
            if len(e.want) and not all(0 <= int(w) < n for w in e.want):
                w = next(int(w) for w in e.want if not 0 <= int(w) < n)
                fail(EINVAL, f"step: request {e.req_id!r} wants logits at place {w} of {n} tokens")
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
            step = self._inputs(entries, fed, fed_rows)
            logits = self.ops.scratch("logits", (max(step.n_logit_rows, 1), self.vocab_size), torch.float32)
            logits = logits[:step.n_logit_rows]
            self._run(step, logits)
            if self.profile is not None:
                self._book_times("prefill" if step.max_q_len > 1 else "decode")
        except BaseException:
            self.ops.abandon()
            for r in reserved:
                mgr.rollback(r)
            for r in admitted:
                mgr.release(r)
            raise
        for e in entries:
            mgr.commit(e.req_id, len(e.tokens))
        self.steps_run += 1
        return logits

    # ---- the common decode step, with less work on the host -----------------------
    def _is_plain_decode(self, entries):
        """Every entry is a known request that brings one token and wants its logits."""
        held = self.manager.held
        try:
            return all(len(e.tokens) == 1 and len(e.want) == 1 and e.want[0] == 0 and e.req_id in held
                       for e in entries)
        except TypeError:
            return False

    def _decode_step(self, entries, fed=None, fed_rows=None):
        """``step`` for entries that pass ``_is_plain_decode``: the same checks, books and arrays,
        built with one pass over the requests instead of several per request."""
        mgr = self.manager
        S = len(entries)
        hs = [mgr.held[e.req_id] for e in entries]
        if len({id(h) for h in hs}) != S:
            fail(EINVAL, "step: a request appears twice")
        tokens = np.fromiter((e.tokens[0] for e in entries), np.int64, S)
        if tokens.min() < 0 or tokens.max() >= self.vocab_size:
            bad = int(tokens[(tokens < 0) | (tokens >= self.vocab_size)][0])
            fail(EINVAL, f"step: token id {bad} is outside the vocabulary of {self.vocab_size}")       # src/model.c:568
        P = mgr.page_tokens
        reserved = []
        try:
            for e, h in zip(entries, hs):
                if h.length % P == 0 or h.length + 1 > mgr.max_context:
                    mgr.reserve(e.req_id, 1)              # a new page in every group, or the error for a full context
                else:
                    h.reserved = 1                        # the token's row lies on a page the request holds
                reserved.append(e.req_id)
            lengths = np.fromiter((h.length for h in hs), np.int32, S)
            slots = np.fromiter((h.slot for h in hs), np.int32, S)
            G = len(mgr.groups)
            offs = lengths % P
            slot_maps = [np.fromiter((h.tables[g][h.length // P] for h in hs), np.int32, S) * P + offs for g in range(G)]
            for m in slot_maps:
                assert m.min() >= 0, "a position about to be written has no page"
            seq_len = lengths + 1
            tokens = tokens.astype(np.int32)
            # Requests come and go, so a serving loop sees every batch size; a graph per size would be
            # captured and hardly ever replayed. Steps of more than BATCH_BUCKET requests are filled up
            # to a multiple of it with rows that belong to no request: row i of them is position i of
            # the storage's spare slot and spare page, which no request's block table names.
            B = self.BATCH_BUCKET
            pad = (-S) % B if S > B and not mgr.state_entries else 0
            if pad > P or S + pad > self.GRAPH_MAX_TOKENS:
                pad = 0
            if pad:
                extra = np.arange(pad, dtype=np.int32)
                spare = np.full(pad, self.storage.pad_slot, np.int32)
                tokens = np.concatenate([tokens, np.zeros(pad, np.int32)])
                lengths = np.concatenate([lengths, extra])
                slots = np.concatenate([slots, spare])
                seq_len = np.concatenate([seq_len, extra + 1])
                slot_maps = [np.concatenate([m, np.int32(page * P) + extra]) for m, page in zip(slot_maps, self.storage.pad_pages)]
            N = S + pad
            rows = np.arange(N, dtype=np.int32)
            q_start = np.arange(N + 1, dtype=np.int32)
            arrays = [tokens, lengths, slots, q_start, slots, seq_len, rows, np.zeros(1, np.int32)] + slot_maps
            moves = (fed[0], as_i32(list(fed_rows)), as_i32(list(fed_rows.values()))) if fed_rows else None
            step = self._upload(arrays, N, N, N, 1, int(seq_len.max()),
                                dict(tokens=tokens, positions=lengths, token_slot=slots, q_start=q_start,
                                     seq_slot=slots, seq_len=seq_len, logit_rows=rows), short=(N, N, 1), moves=moves)
            logits = self.ops.scratch("logits", (N, self.vocab_size), torch.float32)
            self._run(step, logits)
            logits = logits[:S]
            if self.profile is not None:
                self._book_times("decode")
        except BaseException:
            self.ops.abandon()
            for r in reserved:
                mgr.rollback(r)
            raise
        for e in entries:
            mgr.commit(e.req_id, 1)
        self.steps_run += 1
        return logits

    def _run(self, step, logits):
        """The forward pass of the step, eagerly or as a replay of the graph of its shape."""
        decode_only = step.max_q_len == 1 and step.n_tokens <= self.GRAPH_MAX_TOKENS
        if decode_only:
            # The kernels use max_seq_len only to choose how the key range is cut, so a graph
            # captured for a length bucket serves every shorter length too. Steps that run eagerly
            # take the same bucket: a replay and an eager run of a step give the same bits.
            B = self.GRAPH_LEN_BUCKET
            step.max_seq_len = min(-(-step.max_seq_len // B) * B, self.manager.max_context)
        if not (self.use_graphs and decode_only) or self.profile is not None:
            return self.model.forward(self.ops, step, self.storage.views, logits)
        key = (step.n_tokens, step.n_logit_rows, step.max_seq_len)
        stamp = (self.ops.scratch_generation, self.staging.generation)
        hit = self._graphs.get(key)
        if hit is not None and hit[0] == stamp:
            self._graphs[key] = self._graphs.pop(key)        # the dict's order is the order of last use
            hit[1].replay()
            self.graph_replays += 1
            return
        if key not in self._graph_seen:          # first sight: run eagerly, which also sizes the work buffers
            self._graph_seen.add(key)
            return self.model.forward(self.ops, step, self.storage.views, logits)
        memory.note("a captured step")
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.model.forward(self.ops, step, self.storage.views, logits)
        if (self.ops.scratch_generation, self.staging.generation) != stamp:
            fail(EINVAL, "a work buffer moved while a step was captured")
        self._graphs.pop(key, None)
        self._graphs[key] = (stamp, graph)
        while len(self._graphs) > self.GRAPHS_KEPT:
            del self._graphs[next(iter(self._graphs))]
        graph.replay()
        self.graph_replays += 1

    def _inputs(self, entries, fed=None, fed_rows=None):
        mgr = self.manager
        fed_dst, fed_src = [], []
        T = sum(len(e.tokens) for e in entries)
        S = len(entries)
        tokens = np.empty(T, np.int32)
        positions = np.empty(T, np.int32)
        token_slot = np.empty(T, np.int32)
        q_start = np.zeros(S + 1, np.int32)
        seq_slot = np.empty(S, np.int32)
        seq_len = np.empty(S, np.int32)
        rows_of = [None] * S
        slot_maps = [np.empty(T, np.int32) for _ in mgr.groups]
        at = 0
        max_q = max_len = 0
        # Requests with few tokens first (see StepInputs); logits keep the order of the entries.
        few = self._short_rows
        order = sorted(range(S), key=lambda i: len(entries[i].tokens) >= few)
        n_short = n_short_tokens = max_short = 0
        for s, i in enumerate(order):
            e = entries[i]
            h = mgr.held[e.req_id]
            n = len(e.tokens)
            if n < few:
                n_short, n_short_tokens, max_short = n_short + 1, n_short_tokens + n, max(max_short, n)
            tokens[at:at + n] = e.tokens
            if fed_rows and i in fed_rows:
                fed_dst.append(at)
                fed_src.append(fed_rows[i])
            positions[at:at + n] = np.arange(h.length, h.length + n, dtype=np.int32)
            token_slot[at:at + n] = h.slot
            q_start[s + 1] = at + n
            seq_slot[s] = h.slot
            seq_len[s] = h.length + n
            rows_of[i] = [at + int(w) for w in e.want]
            for g in range(len(mgr.groups)):
                slot_maps[g][at:at + n] = mgr.slot_rows(e.req_id, g, h.length, n)
            max_q = max(max_q, n)
            max_len = max(max_len, h.length + n)
            at += n
        rows = as_i32([r for per_entry in rows_of for r in per_entry])
        q_start_long = q_start[n_short:] - n_short_tokens
        arrays = [tokens, positions, token_slot, q_start, seq_slot, seq_len, rows, q_start_long] + slot_maps
        return self._upload(arrays, T, S, len(rows), max_q, max_len,
                            dict(tokens=tokens, positions=positions, token_slot=token_slot, q_start=q_start,
                                 seq_slot=seq_slot, seq_len=seq_len, logit_rows=rows),
                            short=(n_short, n_short_tokens, max_short),
                            moves=(fed[0], as_i32(fed_dst), as_i32(fed_src)) if fed_dst else None)

    def _upload(self, arrays, T, S, R, max_q, max_len, host, short, moves=None):
        """Sends a step's arrays (tokens, positions, token_slot, q_start, seq_slot, seq_len,
        logit_rows, q_start_long, then one slot map per group) and the block-table entries appended
        since the last step; returns the StepInputs. ``short``: number of the leading requests with
        few tokens, their tokens, and the most tokens one of them brings."""
        mgr = self.manager
        # Arrays whose sizes follow from (T, S, R) come first, so that their places in the
        # device buffer are the same for every step of one shape (a captured graph reads them there).
        G = len(mgr.groups)
        dirty = []
        for g in range(G):
            app = mgr.drain_appended(g)
            dirty.append(len(app))
            arrays.append(as_i32([slot * mgr.max_blocks + block for slot, block, _ in app]))
            arrays.append(as_i32([page for _, _, page in app]))
        if moves is not None:                 # tokens that lie on the device: where they go, where they come from
            arrays += [moves[1], moves[2]]
        views = self.staging.upload(arrays)
        step = StepInputs(T, S, R)
        (step.tokens, step.positions, step.token_slot, step.q_start, step.seq_slot, step.seq_len,
         step.logit_rows, step.q_start_long) = views[:8]
        step.max_q_len, step.max_seq_len = max_q, max_len
        step.n_short_seqs, step.n_short_tokens, step.max_short_q_len = short
        step.host = host
        step.rows_in_order = R == T and bool(np.array_equal(host["logit_rows"], np.arange(T)))
        for g in range(G):
            slot_map = views[8 + g]
            idx, val = views[8 + G + 2 * g:10 + G + 2 * g]
            table = self.storage.block_tables[g]
            if dirty[g]:
                self.ops.scatter_i32(table.view(-1), idx, val)
            step.groups.append(GroupInputs(table, slot_map))
        if moves is not None:
            self.ops.move_i32(step.tokens, views[-2], moves[0], views[-1])
        return step

"""The scheduler: admits requests, cuts prompts into portions under a token budget,
decodes, finishes and frees.

The reference serves one request at a time: prefill in chunks of ``--batch`` tokens with
logits only for the last chunk (src/ops.c:788-795), then sample -> check -> feed per step
(src/ops.c:827-893). Here many requests share every step. Per request the order of events
is the reference's: the first token is sampled from the prefill's logits; an end-of-sequence
token is neither reported nor fed (src/ops.c:849); a token sampled at the last allowed step
is reported but not fed (src/ops.c:881); the cap on new tokens is
``min(max_tokens, ctx_max - prompt)`` with stop reason ``length`` or ``ctx`` (src/ops.c:757-758).

Each step:
 1. every running request whose next token is a single decoded token brings it (if there are more
    of them than the token budget, those that waited longest);
 2. what is left of the token budget goes to prompt portions, oldest request first:
    first those already running, then waiting ones, admitted while a state slot is free
    and fewer than ``max_seqs`` are live;
 3. pages for the whole step are checked before it runs. If they do not suffice, prompt
    portions are shrunk or dropped, newest first. If the decoded tokens alone do not fit,
    the most recently admitted running request is preempted: its pages and slot are given
    back, its tokens (prompt and what it generated) are kept, and it waits at the head of
    the queue to be recomputed as a prompt, which starts once pages for all its tokens are
    free again (so it is not thrown out again at once). A request that does not fit even
    alone fails with ERANGE.

The host does not wait for a step's tokens before it enqueues the next step: where the sampler can
leave the chosen tokens on the device (``sample_start``: all rows greedy, or all drawn from their best
k), the next step takes them from there (``Engine.step(..., fed=...)``) and the host reads them
while that step runs. What the host then learns one step late: an end-of-sequence token (the
request ran one step more, whose row is dropped and whose cache goes back with the request).
Steps in which a request is about to end by its length, a prompt's continuations are about to be
forked, or pages are short wait for the tokens first, as do samplers without ``sample_start``.

Several continuations of one prompt (``--n``, src/ops.c:808-825): the prompt is computed once;
when its last portion is done the other continuations are forked from the first one's cache
(whole pages shared), and each samples its own first token from the same logits with its own
seed. A continuation for which no slot or page is free at that moment waits in the queue
and computes the prompt itself.
"""
import itertools
import time
from collections import deque
from dataclasses import dataclass, field

from ..cache import OutOfPages
from ..sampling import Rng, SamplerParams
from ..status import ECANCEL, EINVAL, ENOMEM, ERANGE, EngineError, fail

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass
class Request:
    req_id: object
    prompt: list
    params: SamplerParams = field(default_factory=SamplerParams)
    max_tokens: int = 512                    # src/opts.c:107
    seed: int = 0
    logprobs: int = 0
    eos_ids: tuple = ()
    timeout: float = 0.0                     # seconds, 0 = none
    # ---- state ----
    status: str = WAITING
    tokens: list = None                      # prompt + generated tokens (the next input stream)
    n_fed: int = 0                           # how many of `tokens` are in the cache
    generated: list = field(default_factory=list)
    choices: list = field(default_factory=list)
    stop: str = None                         # eos | length | ctx | cancel | timeout
    error: EngineError = None
    cancel: bool = False
    n_cap: int = 0
    rng: Rng = None
    preemptions: int = 0
    t_submit: float = 0.0
    t_first: float = None                    # when the prompt was done (first logits)
    t_done: float = None
    admitted_at: int = -1                    # admission order, for the preemption choice
    forks: list = field(default_factory=list)     # continuations of the same prompt, forked when it is done
    last_ran: int = -1                       # the step that last held tokens of this request
    pending: int = None                      # its next token is not read yet: row of the sample under way

    @property
    def unfed(self):
        return len(self.tokens) - self.n_fed


PLACEHOLDER = -1         # in Request.tokens: a token that the device has and the host has not read yet


@dataclass
class Inflight:
    """A step's sampling under way: the requests of its rows and the sampler's handle."""
    sampled: list
    started: object


@dataclass
class StepPlan:
    entries: list            # (request, n_tokens, wants_logits)
    preempted: list
    failed: list


class Scheduler:
    def __init__(self, engine, sampler, token_budget=64, max_seqs=None, ctx_max=None, clock=time.monotonic,
                 pipeline=True):
        self.engine, self.sampler = engine, sampler
        self.manager = engine.manager
        self.token_budget = int(token_budget)                          # --batch, src/opts.c:44
        self.max_seqs = min(max_seqs or self.manager.n_slots, self.manager.n_slots)
        self.ctx_max = min(ctx_max or self.manager.max_context, self.manager.max_context)
        if self.token_budget < 1 or self.max_seqs < 1:
            fail(EINVAL, "scheduler: the token budget and max_seqs must be at least 1")
        self.clock = clock
        self.waiting = deque()
        self.running = []
        self.finished = []
        self._admissions = 0
        self.steps = 0
        self.on_token = None          # callback(request, choice)
        self.on_finish = None         # callback(request)
        self.on_prefill = None        # callback(request)
        self.on_step = None           # callback(step number, plan) before the step runs
        self.pipeline = bool(pipeline) and hasattr(sampler, "sample_start")
        self._inflight = None         # the step whose tokens the host has not read yet
        self.steps_ahead = 0          # steps that were enqueued before the tokens of the one before were read

    # ---- submission --------------------------------------------------------
    def submit(self, req, forks=()):
        """Queues ``req``. ``forks`` are further requests with the same prompt (other seeds):
        they do not queue, but start from ``req``'s cache when its prompt is done."""
        for c in forks:
            if list(c.prompt) != list(req.prompt):
                fail(EINVAL, "a fork must have the prompt of the request it is forked from")
            self._prepare(c)
        self._prepare(req)
        req.forks = list(forks)
        self.waiting.append(req)
        return req

    def _prepare(self, req):
        if len(req.prompt) == 0:
            fail(EINVAL, "the prompt is empty")                                     # src/ops.c:752
        if len(req.prompt) >= self.ctx_max:
            fail(ERANGE, f"the prompt has {len(req.prompt)} tokens, --ctx-max is {self.ctx_max}")   # src/ops.c:753-756
        vocab = self.engine.vocab_size
        for t in req.prompt:
            if not 0 <= int(t) < vocab:
                fail(EINVAL, f"token id {t} is outside the vocabulary of {vocab}")  # src/ops.c:582
        if req.max_tokens < 1:
            fail(EINVAL, "--max-tokens must be at least 1")
        req.params.check()
        req.tokens = [int(t) for t in req.prompt]
        req.n_cap = min(req.max_tokens, self.ctx_max - len(req.prompt))             # src/ops.c:757
        req.rng = Rng(req.seed)
        req.status = WAITING
        req.t_submit = self.clock()

    @property
    def idle(self):
        return not self.waiting and not self.running and self._inflight is None

    # ---- planning ------------------------------------------------------------
    def plan(self):
        """Decides what the next step holds. Changes the books only by preempting or failing
        requests that cannot go on; every pass of the loop either returns or removes a
        request from the running set, so it ends."""
        preempted, failed = [], []
        while True:
            entries = self._fill(preempted)
            if entries is not None and (entries or not self.running):
                break
            # The decoded tokens do not fit, or nobody can move: the newest running request yields.
            victim = max(self.running, key=lambda r: r.admitted_at)
            if len(self.running) == 1:
                self._finish(victim, error=EngineError(ERANGE, f"request {victim.req_id!r} does not fit the "
                                                                "cache even alone"))
                failed.append(victim)
            else:
                self._preempt(victim)
                preempted.append(victim)
        if not entries and self.waiting:
            head = self.waiting.popleft()         # nothing runs and the head of the queue cannot start
            self._finish(head, error=EngineError(ERANGE, f"request {head.req_id!r} does not fit the cache "
                                                         "even alone"))
            failed.append(head)
        return StepPlan(entries, preempted, failed)

    def _fill(self, preempted):
        """The entries of a step under the budget and the pages at hand, or None if not even
        the decoded tokens fit."""
        mgr = self.manager
        decode = self._decoders()
        budget = self.token_budget
        if not mgr.can_reserve([(r.req_id, 1) for r in decode]):      # only for those that run
            return None
        entries = [(r, 1, True) for r in decode]
        budget -= len(entries)
        wanted = [(r.req_id, 1) for r, _, _ in entries]
        prefilling = [r for r in self.running if not (r.unfed == 1 and r.n_fed > 0)]
        live = len(self.running)
        free_slots = mgr.n_slots - len(mgr.held)
        # the loop leaves at the first request that has to wait: the queue is walked, never copied
        candidates = itertools.chain(((r, False) for r in prefilling), ((r, True) for r in self.waiting))
        for r, is_new in candidates:
            if budget <= 0:
                break
            if is_new and (live >= self.max_seqs or free_slots <= 0 or r in preempted):
                break
            if is_new and r.preemptions and not mgr.can_reserve(wanted + [(r.req_id, r.unfed)]):
                break                          # a preempted request returns when all it lost fits again
            n = min(r.unfed, budget)
            # shrink the portion to what the pages allow; skip the request if not even one token fits
            while n > 0 and not mgr.can_reserve(wanted + [(r.req_id, n)]):
                n = self._shrink(r, n)
            if n <= 0:
                if is_new:
                    break                      # keep the queue's order: nobody overtakes
                continue
            entries.append((r, n, n == r.unfed))
            wanted.append((r.req_id, n))
            budget -= n
            if is_new:
                live += 1
                free_slots -= 1
        return entries

    def _decoders(self):
        """The running requests that bring one decoded token to the next step."""
        decode = [r for r in self.running if r.unfed == 1 and r.n_fed > 0]
        if len(decode) > self.token_budget:
            # More requests decode than a step may hold tokens (the reference refuses --n above --batch,
            # src/ops.c:810): they take turns, those that waited longest first, so every one advances.
            decode = sorted(decode, key=lambda r: r.last_ran)[:self.token_budget]
        return decode

    def _shrink(self, r, n):
        """The next smaller portion worth trying: one page less."""
        P = self.manager.page_tokens
        held = self.manager.held.get(r.req_id)
        start = held.length if held else 0
        return ((start + n - 1) // P) * P - start        # tokens that end just before the last page touched

    def _preempt(self, r):
        self.engine.release(r.req_id)
        self.running.remove(r)
        r.n_fed = 0
        r.status = WAITING
        r.preemptions += 1
        self.waiting.appendleft(r)

    def _finish(self, r, stop=None, error=None):
        if r.status == RUNNING:
            self.running.remove(r)
            if self.engine.has(r.req_id):
                self.engine.release(r.req_id)
        elif r.status == WAITING and r in self.waiting:
            self.waiting.remove(r)
        r.pending = None
        r.status, r.stop, r.error, r.t_done = FINISHED, stop, error, self.clock()
        self.finished.append(r)
        if self.on_finish:
            self.on_finish(r)
        pending, r.forks = r.forks, []
        for c in pending:                      # the prompt never got done: its other continuations end with it
            self._finish(c, stop=stop, error=error)

    # ---- one step ------------------------------------------------------------
    def step(self):
        """Plans, runs and books one step. Returns the plan (None if there was nothing to do)."""
        now = self.clock()
        # Live requests are polled every step; a long queue is walked every 32nd step only (a request
        # that waits has nothing that a cancellation could stop, it is only reported a little later).
        polled = list(self.running)
        if len(self.waiting) <= 256 or self.steps % 32 == 0:
            polled += list(self.waiting)
        for r in polled:                                                        # src/ops.c:790, 829
            expired = r.timeout > 0 and now - r.t_submit > r.timeout
            if r.cancel or expired:
                if r.t_first is None and r.pending is None:     # still in its prompt: an error, as in the reference
                    self._finish(r, error=EngineError(ECANCEL, "cancelled" if r.cancel else "timeout during prefill"))
                else:
                    self._finish(r, stop="cancel" if r.cancel else "timeout")
        if self._inflight is not None:
            # Tokens are read before the plan where the plan turns on them: a request that is about to end
            # by its length holds pages until its last token is booked; short pages may be freed by an
            # end-of-sequence token that the host has not seen.
            if not self.running or any(r.unfed == 0 for r in self.running) \
                    or not self.manager.can_reserve([(r.req_id, 1) for r in self._decoders()]):
                self._land()
        if self.idle:
            return None
        plan = self.plan()
        if not plan.entries:
            self._land()
            return plan
        for r, _, _ in plan.entries:
            if r.status == WAITING:
                self.waiting.remove(r)
                r.status = RUNNING
                r.admitted_at = self._admissions
                self._admissions += 1
                self.running.append(r)
        if self.on_step:
            self.on_step(self.steps, plan)
        step_entries = [(r.req_id, r.tokens[r.n_fed:r.n_fed + n], [n - 1] if want else [])
                        for r, n, want in plan.entries]
        fed = None
        if self._inflight is not None:
            rows = {i: r.pending for i, (r, n, _) in enumerate(plan.entries) if r.pending is not None}
            if rows:
                fed = (self._inflight.started.device_tokens, rows)
                self.steps_ahead += 1
        logits = self.engine.step(step_entries, fed=fed) if fed else self.engine.step(step_entries)
        self.steps += 1
        sampled = [r for r, n, want in plan.entries if want]
        for r, n, _ in plan.entries:
            r.n_fed += n
            r.last_ran = self.steps
        self._land()                  # the step before: its tokens are read while this one runs
        if sampled:
            t0 = time.perf_counter()
            wants = [(r.params, r.rng, r.logprobs) for r in sampled]
            ahead = self.pipeline and not any(r.forks and r.t_first is None for r in sampled)
            started = self.sampler.sample_start(logits, wants) if ahead else None
            if started is not None and started.device_tokens is not None:
                self._inflight = Inflight(sampled, started)
                for i, r in enumerate(sampled):
                    # a request that goes on decoding gets its next token's place now; one that this token
                    # ends (by its length) or that has ended meanwhile only has the token booked later
                    if r.status == RUNNING and len(r.generated) + 1 < r.n_cap:
                        r.tokens.append(PLACEHOLDER)
                        r.pending = i
            else:
                choices = started.finish() if started is not None else self.sampler.sample(logits, wants)
                for i, (r, ch) in enumerate(zip(sampled, choices)):
                    if r.status != RUNNING:
                        continue              # ended by a token of the step before, which the host has just read
                    forked = self._fork(r, logits[i:i + 1]) if r.forks and r.t_first is None else []
                    self._accept(r, ch)
                    for c, cch in forked:
                        self._accept(c, cch)
            book = getattr(self.engine, "profile", None)
            if book is not None:               # sampling is timed on the host, as in src/ops.c:845-847
                stage = book["prefill" if any(n > 1 for _, n, _ in plan.entries) else "decode"]
                stage["sample"] = stage.get("sample", 0.0) + (time.perf_counter() - t0) * 1e3
        return plan

    def _land(self):
        """Reads the tokens of the step whose sampling is under way and books them."""
        flight, self._inflight = self._inflight, None
        if flight is None:
            return
        choices = flight.started.finish()
        for i, (r, ch) in enumerate(zip(flight.sampled, choices)):
            if r.status == FINISHED:
                continue                      # cancelled, or ended while this token was on its way
            self._accept(r, ch, placed=r.pending == i)

    def _fork(self, r, row):
        """``r``'s prompt is done: its other continuations take its cache and draw their first
        token from the same logits. Returns [(request, choice)] of those that could be forked."""
        pending, r.forks = r.forks, []
        out = []
        for c in pending:
            try:
                if len(self.running) >= self.max_seqs:
                    raise OutOfPages("as many sequences are live as may be")
                self.engine.fork(r.req_id, c.req_id)
            except EngineError as e:
                if e.code != ENOMEM:
                    raise
                self.waiting.append(c)         # no room now: it computes the prompt itself later
                continue
            c.status, c.n_fed = RUNNING, r.n_fed
            c.admitted_at = self._admissions
            self._admissions += 1
            self.running.append(c)
            out.append((c, self.sampler.sample(row, [(c.params, c.rng, c.logprobs)])[0]))
        return out

    def _accept(self, r, ch, placed=False):
        """Books a sampled token. ``placed``: the token already has its place at the end of ``r.tokens``
        (and may have been fed from the device); the place is filled, or dropped with the request."""
        r.pending = None
        if r.t_first is None:
            r.t_first = self.clock()
            if self.on_prefill:
                self.on_prefill(r)
        if ch.token in r.eos_ids:                                              # src/ops.c:849
            if placed:
                r.tokens.pop()
            return self._finish(r, stop="eos")
        r.generated.append(ch.token)
        r.choices.append(ch)
        if self.on_token:
            self.on_token(r, ch)
        if len(r.generated) >= r.n_cap:                                        # src/ops.c:881, 758
            return self._finish(r, stop="length" if r.n_cap == r.max_tokens else "ctx")
        if placed:
            r.tokens[-1] = ch.token
        else:
            r.tokens.append(ch.token)

    def run(self):
        """Steps until every submitted request is finished; returns them in finishing order."""
        while not self.idle:
            self.step()
        return self.finished

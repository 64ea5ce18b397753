"""The scheduler's decisions (no GPU): a stand-in engine with the real cache manager, and a
stand-in sampler that follows a script."""
import pytest

from hf_cpu_amd.cache import CacheManager
from hf_cpu_amd.engine.scheduler import Request, Scheduler
from hf_cpu_amd.parts import PagedKV
from hf_cpu_amd.sampling import Choice, SamplerParams
from hf_cpu_amd.status import EngineError


class FakeEngine:
    """Books pages like the real engine; 'logits' are the list of (request, position) wanted."""

    def __init__(self, n_pages=8, page=4, slots=4, ctx=64, window=0, vocab=100):
        self.manager = CacheManager([PagedKV(4, 4, 0), PagedKV(4, 4, window)], page, n_pages, slots, ctx)
        self.vocab_size = vocab
        self.log = []
        self.fed_steps = 0

    def has(self, r):
        return r in self.manager.held

    def release(self, r):
        self.manager.release(r)

    def fork(self, src, new):
        self.manager.fork(src, new)
        self.log.append([("fork", src, new)])

    def step(self, entries, fed=None):
        m = self.manager
        if fed is not None:
            self.fed_steps += 1
            assert all(len(entries[i][1]) == 1 for i in fed[1])
        for r, toks, want in entries:
            if fed is None or entries.index((r, toks, want)) not in fed[1]:
                assert all(t >= 0 for t in toks), "a token that was never read went to the engine as if known"
        for r, toks, want in entries:
            if r not in m.held:
                m.admit(r)
            m.reserve(r, len(toks))
        rows = []
        for r, toks, want in entries:
            rows += [(r, m.held[r].length + w) for w in want]
            m.commit(r, len(toks))
        self.log.append([(r, len(t), list(w)) for r, t, w in entries])
        m.check()
        return rows

    @property
    def shape(self):
        return None


class Rows(list):
    @property
    def shape(self):
        return (len(self), 0)


class ScriptSampler:
    """Token = 10 + number of tokens generated so far, or what ``script[req]`` says."""

    def __init__(self, script=None):
        self.script = script or {}
        self.count = {}

    def sample(self, logits, wants):
        assert len(logits) == len(wants)
        out = []
        for (req, pos), _ in zip(logits, wants):
            i = self.count.get(req, 0)
            self.count[req] = i + 1
            seq = self.script.get(req)
            out.append(Choice(seq[i] if seq and i < len(seq) else 10 + i))
        return out


def greedy():
    return SamplerParams(temp=0.0)


def make(budget=8, **kw):
    eng = FakeEngine(**kw)
    return eng, Scheduler(eng, ScriptSampler(), token_budget=budget)


def test_prompt_is_cut_into_portions_under_the_budget():
    eng, s = make(budget=8, n_pages=16)
    r = s.submit(Request("a", list(range(19)), greedy(), max_tokens=3))
    s.run()
    assert eng.log[:3] == [[("a", 8, [])], [("a", 8, [])], [("a", 3, [2])]]       # logits only for the last portion
    assert eng.log[3:] == [[("a", 1, [0])], [("a", 1, [0])]]
    assert r.generated == [10, 11, 12] and r.stop == "length"
    # the token sampled at the last allowed step is reported but never fed (src/ops.c:881)
    assert sum(n for step in eng.log for _, n, _ in step) == 19 + 2
    assert not eng.manager.held and all(p.n_held == 0 for p in eng.manager.pools)


def test_decode_tokens_go_first_and_share_steps_with_prompt_portions():
    eng, s = make(budget=8, n_pages=32)
    a = s.submit(Request("a", [1, 2, 3], greedy(), max_tokens=4))
    s.step()
    b = s.submit(Request("b", list(range(20)), greedy(), max_tokens=2))
    s.step()
    assert eng.log[1] == [("a", 1, [0]), ("b", 7, [])]       # one decoded token, the rest of the budget to b
    s.step()
    assert eng.log[2] == [("a", 1, [0]), ("b", 7, [])]
    s.run()
    assert a.generated == [10, 11, 12, 13] and b.generated == [10, 11]
    assert a.stop == b.stop == "length"


def test_admission_is_fifo_and_bounded_by_slots():
    eng, s = make(budget=64, n_pages=32, slots=2)
    rs = [s.submit(Request(i, [1, 2, 3, 4], greedy(), max_tokens=2 + i)) for i in range(4)]
    s.step()
    assert [r for r, _, _ in eng.log[0]] == [0, 1]             # two slots
    s.run()
    order = [r.req_id for r in s.finished]
    assert order == [0, 1, 2, 3]
    first_seen = {}
    for i, step in enumerate(eng.log):
        for r, _, _ in step:
            first_seen.setdefault(r, i)
    assert first_seen[2] < first_seen[3] or first_seen[2] == first_seen[3]
    assert first_seen[2] > first_seen[1]


def test_eos_is_neither_reported_nor_fed():
    eng = FakeEngine()
    s = Scheduler(eng, ScriptSampler({"a": [5, 6, 99, 7]}), token_budget=8)
    seen = []
    s.on_token = lambda r, ch: seen.append(ch.token)
    r = s.submit(Request("a", [1, 2], greedy(), max_tokens=10, eos_ids=(99,)))
    s.run()
    assert r.generated == [5, 6] and seen == [5, 6] and r.stop == "eos"        # src/ops.c:849
    assert sum(n for step in eng.log for _, n, _ in step) == 2 + 2


def test_context_cap_gives_stop_ctx():
    eng, s = make(budget=8, ctx=8, n_pages=8)
    r = s.submit(Request("a", [1, 2, 3, 4, 5], greedy(), max_tokens=10))
    s.run()
    assert len(r.generated) == 3 and r.stop == "ctx"           # min(max_tokens, ctx_max - prompt), src/ops.c:757-758
    with pytest.raises(EngineError) as e:
        s.submit(Request("b", list(range(8)), greedy()))
    assert e.value.code == "ERANGE" and "ctx-max" in str(e.value)
    with pytest.raises(EngineError) as e:
        s.submit(Request("c", [], greedy()))
    assert e.value.code == "EINVAL"
    with pytest.raises(EngineError) as e:
        s.submit(Request("d", [1, 100], greedy()))
    assert e.value.code == "EINVAL" and "vocabulary" in str(e.value)


def test_prompt_portion_shrinks_to_the_pages_left():
    eng, s = make(budget=64, n_pages=6, page=4)                # 24 tokens of pages
    a = s.submit(Request("a", list(range(13)), greedy(), max_tokens=8))
    s.step()                                                   # a holds 4 pages
    b = s.submit(Request("b", list(range(30)), greedy(), max_tokens=1))
    s.step()
    # a decodes (position 13 fits its 4th page); b gets the two pages left: 8 tokens
    assert eng.log[1] == [("a", 1, [0]), ("b", 8, [])]
    s.step()
    assert eng.log[2] == [("a", 1, [0])]                       # nothing left for b, a goes on


def test_preemption_when_decode_runs_out_of_pages():
    eng, s = make(budget=64, n_pages=4, page=4)                # 16 tokens of pages
    a = s.submit(Request("a", list(range(7)), greedy(), max_tokens=6))
    b = s.submit(Request("b", list(range(7)), greedy(), max_tokens=6))
    s.step()                                                   # both prompts: 2 pages each, pool full
    assert eng.manager.pools[0].n_free == 0
    s.step()                                                   # both decode inside their pages (positions 7)
    assert [r for r, _, _ in eng.log[1]] == ["a", "b"]
    plan = s.step()                                            # position 8 needs a page each: none free
    assert [r.req_id for r in plan.preempted] == ["b"]         # the most recently admitted goes
    assert b.status == "waiting" and b.n_fed == 0 and b.preemptions == 1 and b.generated == [10, 11]
    assert eng.log[2] == [("a", 1, [0])]
    s.run()
    assert a.generated == [10, 11, 12, 13, 14, 15] and a.stop == "length"
    # b was recomputed as a prompt of 7 + 2 tokens and went on where it was
    assert b.generated == [10, 11, 12, 13, 14, 15] and b.stop == "length"
    recompute = [e for step in eng.log for e in step if e[0] == "b" and e[1] == 9]
    assert recompute == [("b", 9, [8])]
    assert not eng.manager.held and all(p.n_held == 0 for p in eng.manager.pools)


def test_request_that_fits_not_even_alone_fails_with_erange():
    eng, s = make(budget=64, n_pages=2, page=4, ctx=64)        # 8 tokens of pages
    r = s.submit(Request("a", list(range(5)), greedy(), max_tokens=20))
    s.run()
    assert r.error is not None and r.error.code == "ERANGE" and len(r.generated) == 4
    assert not eng.manager.held
    big = s.submit(Request("b", list(range(20)), greedy(), max_tokens=2))
    s.run()
    # its prompt is fed in what the pool allows, then it cannot go on
    assert big.error is not None and big.error.code == "ERANGE"
    assert not eng.manager.held and all(p.n_held == 0 for p in eng.manager.pools)


def test_cancel_and_timeout():
    now = [0.0]
    eng = FakeEngine(n_pages=32)
    s = Scheduler(eng, ScriptSampler(), token_budget=4, clock=lambda: now[0])
    b = s.submit(Request("b", [1, 2], greedy(), max_tokens=50, timeout=5.0))
    a = s.submit(Request("a", list(range(10)), greedy(), max_tokens=50, timeout=5.0))
    s.step()
    s.step()
    assert eng.log == [[("b", 2, [1]), ("a", 2, [])], [("b", 1, [0]), ("a", 3, [])]]
    assert b.t_first is not None and a.t_first is None
    now[0] = 6.0
    s.step()
    assert a.error.code == "ECANCEL" and a.stop is None       # expiry during the prompt is an error
    assert b.stop == "timeout" and b.error is None and len(b.generated) >= 1
    c = s.submit(Request("c", [1], greedy(), max_tokens=50))
    s.step()
    s.step()
    c.cancel = True
    s.step()
    assert c.stop == "cancel" and not eng.manager.held


def test_windowed_group_frees_pages_for_others():
    eng, s = make(budget=4, n_pages=5, page=4, window=4, ctx=64)
    r = s.submit(Request("a", list(range(3)), greedy(), max_tokens=30))
    s.run()
    # 33 tokens need 9 pages in the full group: it fails there, but the windowed group never held more than 3
    assert eng.manager.pools[1].high_water <= 3
    assert r.error is not None and r.error.code == "ERANGE"


def test_continuations_of_one_prompt_fork_from_its_cache():
    eng, s = make(budget=8, n_pages=16, slots=4)
    fam = [Request(f"c{i}", list(range(10)), greedy(), max_tokens=3, seed=i) for i in range(3)]
    s.submit(fam[0], forks=fam[1:])
    assert list(s.waiting) == [fam[0]]                 # the others do not queue
    s.step()
    assert eng.log[-1] == [("c0", 8, [])]
    s.step()                                           # the prompt's end: the others take its cache
    assert eng.log[-3:] == [[("c0", 2, [1])], [("fork", "c0", "c1")], [("fork", "c0", "c2")]]
    assert [r.req_id for r in s.running] == ["c0", "c1", "c2"] and all(len(r.generated) == 1 for r in fam)
    assert all(r.n_fed == 10 for r in fam)
    m = eng.manager
    assert m.held["c1"].tables[0][:2] == m.held["c0"].tables[0][:2] and m.held["c1"].tables[0][2] != m.held["c0"].tables[0][2]
    s.step()
    assert eng.log[-1] == [("c0", 1, [0]), ("c1", 1, [0]), ("c2", 1, [0])]      # the prompt was computed once
    s.run()
    assert all(r.stop == "length" and len(r.generated) == 3 for r in fam)
    assert all(p.n_held == 0 for p in m.pools)
    m.check()


def test_a_continuation_without_room_computes_the_prompt_itself():
    eng, s = make(budget=16, n_pages=16, slots=2)
    fam = [Request(f"c{i}", list(range(6)), greedy(), max_tokens=2, seed=i) for i in range(3)]
    s.submit(fam[0], forks=fam[1:])
    s.step()                                           # two slots: c1 forks, c2 has to wait
    assert [r.req_id for r in s.running] == ["c0", "c1"] and list(s.waiting) == [fam[2]]
    s.run()
    assert all(r.stop == "length" and len(r.generated) == 2 for r in fam)
    assert any(step == [("c2", 6, [5])] or ("c2", 6, [5]) in step for step in eng.log)
    eng.manager.check()


def test_continuations_end_with_a_prompt_that_fails():
    eng, s = make(budget=8, n_pages=2, page=4, ctx=64)
    fam = [Request(f"c{i}", list(range(20)), greedy(), max_tokens=2, seed=i) for i in range(2)]
    s.submit(fam[0], forks=fam[1:])
    s.run()
    assert all(r.error is not None and r.error.code == "ERANGE" for r in fam)
    with pytest.raises(EngineError):
        s.submit(Request("x", [1, 2], greedy()), forks=[Request("y", [1, 3], greedy())])


def test_a_cancellation_deep_in_a_long_queue_is_seen_within_32_steps():
    """More than 256 requests waiting: the queue is polled every 32nd step only; a request cancelled
    while it waits ends with ECANCEL before it is ever admitted."""
    eng, s = make(budget=8, n_pages=64, slots=2)
    rs = [s.submit(Request(i, [1, 2, 3], greedy(), max_tokens=40)) for i in range(400)]
    s.step()
    victim = rs[350]
    victim.cancel = True
    for _ in range(33):
        s.step()
    assert victim.error is not None and victim.error.code == "ECANCEL" and victim.admitted_at == -1
    assert all(350 not in [r for r, _, _ in step] for step in eng.log)


def test_more_decoding_requests_than_the_token_budget_take_turns():
    """Four requests decode under a budget of 3 tokens a step: every step holds three decoded tokens,
    nobody waits more than one step in a row, pages are reserved only for those that run, and every
    request ends with the tokens it gets alone."""
    eng, sch = make(budget=3, n_pages=16, page=4, slots=4, ctx=64)
    reqs = [sch.submit(Request(f"r{i}", [1, 2, 3][:1 + i % 3], greedy(), max_tokens=9)) for i in range(4)]
    sch.run()
    assert all(r.stop == "length" and len(r.generated) == 9 for r in reqs)
    assert all(r.generated == [10 + i for i in range(9)] for r in reqs)          # the script's tokens, in order
    decode_steps = [s for s in eng.log if all(n == 1 for _, n, _ in s) and len(s) > 1]
    full = [s for s in decode_steps if len(s) == 3]
    assert len(full) >= 8
    for r in reqs:                               # between its first and its last step nobody waits two steps in a row
        ran = [i for i, s in enumerate(eng.log) if any(e[0] == r.req_id for e in s)]
        assert max(b - a for a, b in zip(ran, ran[1:])) <= 2, (r.req_id, ran)
    assert not eng.manager.held
    # Three requests at a page's edge, two free pages, a budget of two: pages are asked for the two that
    # run, not for all three (which would not fit and cost one of them its cache).
    eng2, sch2 = make(budget=16, n_pages=5, page=4, slots=3, ctx=12)
    rs = [sch2.submit(Request(f"q{i}", [1, 2, 3], greedy(), max_tokens=3)) for i in range(3)]
    sch2.step()
    sch2.step()
    assert [eng2.manager.held[r.req_id].length for r in rs] == [4, 4, 4] and eng2.manager.pools[0].n_free == 2
    sch2.token_budget = 2
    sch2.run()
    assert all(r.error is None and len(r.generated) == 3 for r in rs) and sum(r.preemptions for r in rs) == 0


class AheadSampler(ScriptSampler):
    """The script sampler with the interface that leaves tokens "on the device": the choices exist at
    once, but the scheduler may only look at them through ``finish``."""

    def sample_start(self, logits, wants):
        choices = self.sample(logits, wants)

        class Started:
            device_tokens = object()

            def finish(self):
                return choices
        return Started()


@pytest.mark.parametrize("seed", range(12))
def test_steps_enqueued_ahead_give_what_steps_in_turn_give(seed):
    """Random workloads (prompt lengths, caps, end-of-sequence tokens at scripted places, a pool that is
    too small, a budget below the number of decoders) served with the next step enqueued before the
    last one's tokens are read, and served in turn: every request ends with the same tokens and the
    same reason, nothing stays held, and steps did run ahead."""
    import random
    rnd = random.Random(seed)
    n_req = rnd.randint(3, 9)
    spec = []
    for i in range(n_req):
        n_prompt, cap = rnd.randint(1, 14), rnd.randint(1, 12)
        script = [10 + j for j in range(cap)]
        if rnd.random() < 0.5:
            script[rnd.randrange(cap)] = 99                     # the end-of-sequence token somewhere
        spec.append((f"r{i}", list(range(1, n_prompt + 1)), cap, script))
    kw = dict(n_pages=rnd.choice([6, 9, 40]), page=4, slots=rnd.choice([2, 4]), ctx=48)
    budget = rnd.choice([2, 5, 16])
    outcomes = []
    for ahead in (False, True):
        eng = FakeEngine(**kw)
        sampler = (AheadSampler if ahead else ScriptSampler)({name: script for name, _, _, script in spec})
        sch = Scheduler(eng, sampler, token_budget=budget)
        reqs = [sch.submit(Request(name, prompt, greedy(), max_tokens=cap, eos_ids=(99,))) for name, prompt, cap, _ in spec]
        sch.run()
        eng.manager.check()
        assert not eng.manager.held and sch.idle
        outcomes.append([(r.req_id, r.generated, r.stop, r.error.code if r.error else None) for r in reqs])
        if ahead:
            assert sch.steps_ahead == eng.fed_steps
            assert all(t != -1 for r in reqs for t in r.tokens)
            ran_ahead = sch.steps_ahead
    assert outcomes[0] == outcomes[1]
    assert ran_ahead > 0 or all(len(g) <= 1 for _, g, _, _ in outcomes[0])


def test_the_early_read_looks_at_the_decoders_that_will_run():
    """More decoders than the budget, a pool that is almost full, and an end-of-sequence token that the host
    has not read yet: whether the tokens in flight must be read before planning is decided on the decoders
    that the plan will pick (those that waited longest), not on the first ones in running order. Otherwise
    the plan finds its own set short of a page and throws the newest request out, although the token in
    flight frees the pages that are missing."""
    for la, lb, lc, n_pages, low_at, eos_at, who in ((1, 1, 1, 5, 2, 4, 1), (1, 1, 3, 4, 1, 2, 1), (1, 1, 1, 5, 3, 5, 0)):
        eng = FakeEngine(n_pages=n_pages, page=4, slots=3, ctx=32)
        script = {f"r{i}": [10 + j for j in range(12)] for i in range(3)}
        script[f"r{who}"][eos_at] = 99
        sch = Scheduler(eng, AheadSampler(script), token_budget=16)
        reqs = [sch.submit(Request(f"r{i}", list(range(1, n + 1)), greedy(), max_tokens=8, eos_ids=(99,)))
                for i, n in enumerate((la, lb, lc))]
        for _ in range(low_at):
            sch.step()
        sch.token_budget = 2
        sch.run()
        assert all(r.error is None for r in reqs) and sum(r.preemptions for r in reqs) == 0
        assert reqs[who].stop == "eos" and len(reqs[who].generated) == eos_at
        assert all(r.stop == "length" and r.generated == [10 + j for j in range(8)] for r in reqs if r is not reqs[who])
        assert sch.steps_ahead > 0 and not eng.manager.held

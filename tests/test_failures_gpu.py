"""Allocation failures, injected on the host: the n-th allocation the engine asks for fails, for
every n that a request meets (the reference's sweep: ``HFC_FAIL_AFTER`` in tests/e2e.pl:175-179 over
src/mem.c:12-30). Every request still ends with ``@done status=ok|error``, nothing is left held,
and what follows a failed step is right. Nothing here makes the GPU fault: the allocation is
refused before it is made."""
import io
import os
import subprocess
import sys

import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 5e-6, "bfloat16": 2e-2}


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    return helpers.make_model_dir(str(tmp_path_factory.mktemp("failA")), helpers.CONFIG_A, seed=3)


def _events(text):
    evs = []
    for line in text.splitlines():
        if line.startswith("@"):
            name, _, rest = line[1:].partition(" ")
            evs.append((name, dict(p.split("=", 1) for p in rest.split(" ") if "=" in p)))
    return evs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_allocation_of_a_generate_request_may_fail(gpu, model_a, dtype):
    """The command line's request loop in this process, a fresh session for every n: model load,
    cache storage, work buffers, staging, sampler outputs and graph captures all pass the counter."""
    from hf_cpu_amd import memory
    from hf_cpu_amd.cli import main as M
    from hf_cpu_amd.cli import opts as O
    from hf_cpu_amd.cli.proto import Out
    so = O.defaults()
    O.apply(so, ["--dtype", dtype, "--ctx-max", "128", "--page-size", "16", "--max-seqs", "4", "--log-level", "error",
                 "--batch", "8"])
    words = ["--model", model_a, "--prompt-ids", "1 2 3 4 5 6 7 8 9 10 11", "--temp", "0.7", "--seed", "5",
             "--max-tokens", "6", "--n", "2", "--logprobs", "2"]
    ok_tokens, outcomes, n = None, [], 0
    while True:
        n += 1
        stream = io.StringIO()
        cli = M.Cli(dict(so), Out(stream))
        before = memory.allocations()
        memory.fail_after(n)
        try:
            good = cli.run_request(M.effective(so, words))
        finally:
            memory.fail_after(0)
        asked = memory.allocations() - before
        ev = _events(stream.getvalue())
        assert ev[0][0] == "begin" and ev[-1][0] == "done", ev[-3:]
        done = ev[-1][1]
        assert done["status"] == ("ok" if good else "error")
        toks = [(e[1].get("seq"), e[1]["id"]) for e in ev if e[0] == "token"]
        if cli.session is not None:
            mgr = cli.session.engine.manager
            mgr.check()
            assert not mgr.held and all(p.n_held == 0 for p in mgr.pools)
        if good:
            ok_tokens = ok_tokens or toks
            assert toks == ok_tokens                     # a run in which nothing failed gives the same tokens
        else:
            assert done["code"] == "ENOMEM" and "injected" in stream.getvalue()
        outcomes.append(good)
        if asked < n:                                    # the request asked for fewer allocations than n: all swept
            break
        assert n < 400, "the request never stopped allocating"
    assert outcomes[-1] and not all(outcomes), outcomes
    assert n > 20, f"only {n} allocations were swept"
    print(f"{dtype}: {n - 1} allocations swept, {outcomes.count(False)} failed requests")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_failed_step_leaves_no_trace_in_a_mixed_trace(gpu, tmp_path, dtype):
    """A mixed trace (portions beside decoded tokens, pages used again) in which the n-th allocation
    fails, for every n: if the engine could not be built it is built again; a step that failed is run
    again, and every logit of the trace equals the plain implementation's."""
    import hf_cpu_amd
    from hf_cpu_amd import memory
    from hf_cpu_amd.status import EngineError
    cfg = helpers.CONFIG_B
    d = helpers.make_model_dir(str(tmp_path / "m"), cfg, seed=8)
    reqs = helpers.random_requests(cfg, [1, 40, 77, 23], seed=2)
    want = helpers.plain_logits(d, reqs)
    steps = helpers.trace_mixed(reqs, seed=4)
    places = helpers.wanted_places(steps)
    max_tokens = helpers.max_live_tokens(steps)
    n, failed_in_step = 0, 0
    while True:
        n += 1
        before = memory.allocations()
        memory.fail_after(n)
        engine = None
        try:
            try:
                engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=helpers.PAGE["B"], max_tokens=max_tokens,
                                                max_seqs=4)
            except EngineError as e:
                assert e.code == "ENOMEM" and "injected" in e.msg
                memory.fail_after(0)
                engine = hf_cpu_amd.load_engine(d, dtype=dtype, page_tokens=helpers.PAGE["B"], max_tokens=max_tokens,
                                                max_seqs=4)
            got = {}
            for s in steps:
                entries = [(e["id"], e["tokens"], e["want"]) for e in s["entries"]]
                held = {r: engine.length(r) for r in engine.manager.held}
                try:
                    logits = engine.step(entries)
                except EngineError as e:
                    assert e.code == "ENOMEM" and "injected" in e.msg
                    failed_in_step += 1
                    engine.manager.check()
                    assert {r: engine.length(r) for r in engine.manager.held} == held      # as before the step
                    logits = engine.step(entries)
                if s["step"] in places:
                    rows = logits.float().cpu().numpy()
                    for row, key in zip(rows, places[s["step"]]):
                        got[key] = row.copy()
                for r in s["end"]:
                    engine.release(r)
        finally:
            memory.fail_after(0)
        helpers.compare(got, want, TOL[dtype], f"B {dtype} with allocation {n} failing")
        engine.manager.check()
        assert not engine.manager.held
        if memory.allocations() - before < n:
            break
        assert n < 400
    assert failed_in_step > 0, "no allocation failed inside a step"
    print(f"{dtype}: {n - 1} allocations swept, {failed_in_step} failed inside a step")


def test_the_environment_variable_fails_an_allocation_of_the_program(gpu, model_a):
    """``HFAMD_FAIL_AFTER`` as the reference's ``HFC_FAIL_AFTER``: the program ends by itself (no signal),
    with the error event and exit code 1; without the variable the same command succeeds."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "hfamd"), "--stdin-mode", "none", "--dtype", "float32", "--ctx-max", "128",
           "--page-size", "16", "--max-seqs", "2", "--log-level", "error", "--model", model_a, "--prompt-ids", "1 2 3 4 5",
           "--temp", "0", "--max-tokens", "3"]
    for n, want_rc in ((7, 1), (0, 0)):
        env = dict(os.environ, HFAMD_FAIL_AFTER=str(n))
        r = subprocess.run(cmd, env=env, capture_output=True, text=True, timeout=300)
        assert r.returncode == want_rc, (r.returncode, r.stderr[-500:])
        done = [e for e in _events(r.stdout) if e[0] == "done"]
        assert len(done) == 1 and done[0][1]["status"] == ("error" if n else "ok")
        if n:
            assert done[0][1]["code"] == "ENOMEM"

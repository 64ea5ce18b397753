"""The command line: ``hfamd [options]``, requests on stdin, events on stdout, logs on stderr.

Structure after the reference: ``main`` layers defaults < settings < command line
(src/main.c:171-181) and runs one request (``--stdin-mode none``) or a loop over records or
lines (src/main.c:54-153); every request answers ``@begin ... @done status=ok|error``
(src/ops.c:1042-1073); ``generate`` reports ``@prompt``, ``@prefill``, ``@token``, ``@gen``
(src/ops.c:783, 799-804, 852-864, 912-919). The model stays loaded between requests
(src/ops.c:532-561). Exit codes: 0, 1 (failed single request or closed stdout), 2 (startup
option error), 130 (signal) (src/main.c:175-204).
"""
import os
import signal
import sys
import time

from ..status import EINVAL, ENOTSUP, EngineError, fail
from . import opts as O
from .proto import Out, Reader

LEVELS = ("error", "warn", "info", "debug")


class Cli:
    def __init__(self, session_opts, out):
        self.opts = session_opts
        self.out = out
        self.session = None
        self.requests = 0
        self.errors = 0
        self.cancel = False
        self.busy = False
        self.current = []              # scheduler requests of the running generate

    def log(self, level, msg):
        if LEVELS.index(level) <= LEVELS.index(self.opts["log-level"]):
            print(f"{level} {msg}", file=sys.stderr, flush=True)

    # ---- the resident model ---------------------------------------------------
    def resident(self, eff):
        from ..session import Session
        if not eff["model"]:
            fail(EINVAL, f"{eff['op']} needs --model PATH")
        path = eff["model"]
        cfg = os.path.join(path, "config.json")
        try:
            st = os.stat(cfg)
        except OSError as e:
            from ..status import EIO
            fail(EIO, f"cannot read {cfg}: {e.strerror}")
        ident = (os.path.abspath(path), st.st_size, st.st_mtime, eff["random-weights"], eff["window"])
        if self.session is not None and self.session.cli_identity == ident:
            return self.session
        self.session = None
        so = self.opts
        # the window of config.json replaced (0: no window); the architecture's configuration class knows its keys
        over = None if eff["window"] is None else {"window": eff["window"]}
        if eff["random-weights"] is not None:
            from ..config import read_config
            model, seed = read_config(path, over), eff["random-weights"]
        else:
            model, seed = path, 0
        t0 = time.monotonic()
        s = Session(model, dtype=so["dtype"], ctx_max=so["ctx-max"], batch=so["batch"], page_size=so["page-size"],
                    max_seqs=so["max-seqs"], kv_tokens=so["kv-tokens"] or None, seed=seed, model_options=over)
        s.cli_identity = ident
        self.log("info", f"model={path} dtype={so['dtype']} load_ms={(time.monotonic() - t0) * 1e3:.0f} "
                         f"kv_bytes={s.engine.storage.nbytes()}")
        self.session = s
        return s

    # ---- operations -----------------------------------------------------------
    def op_echo(self, eff):
        """Reports the effective options (protocol testing, src/ops.c:410-464)."""
        self.out.event("echo", **{k.replace("-", "_"): eff[k] for k in sorted(eff) if eff[k] is not None})

    def op_generate(self, eff):
        s = self.resident(eff)
        if eff["prompt-ids"] is None:
            fail(ENOTSUP, "there is no tokenizer: give the prompt as --prompt-ids")
        prompts = [parse_ids(p, s.model.vocab_size) for p in eff["prompt-ids"].split(";")]
        nseq = len(prompts) * eff["n"]
        multi = nseq > 1
        top_n = min(eff["logprobs"], 64)
        eos = None if eff["eos-ids"] is None else tuple(parse_ids(eff["eos-ids"], s.model.vocab_size))
        self.out.event("prompt", tokens=sum(len(p) for p in prompts), sequences=nseq)
        t0 = time.monotonic()
        state = {"prefilled": 0, "t_dec0": None}

        def seq_pairs(seq):
            return {"seq": seq} if multi else {}

        def on_prefill(seq, r):
            state["prefilled"] += 1
            if state["prefilled"] == nseq or not multi:
                dt = time.monotonic() - t0
                ntok = sum(len(p) for p in prompts)        # each prompt is computed once, whatever --n
                self.out.event("prefill", tokens=ntok, cached=0, ms=f"{dt * 1e3:.1f}",
                               tok_per_s=f"{ntok / dt if dt > 0 else 0:.2f}",
                               kv_bytes=s.engine.storage.nbytes())
            if state["t_dec0"] is None:
                state["t_dec0"] = time.monotonic()

        def on_token(seq, pos, ch):
            pairs = dict(seq_pairs(seq), pos=pos, id=ch.token)
            if top_n:
                pairs["logprob"] = f"{ch.logprob:.6f}"
                pairs["top"] = " ".join(f"{t}:{lp:.6f}" for t, lp in ch.top)
            self.out.event("token", **pairs)

        try:
            self.busy = True
            if eff["profile"]:
                s.engine.profile_start()
            gens = self._run_generate(s, prompts, eff, eos, on_token, on_prefill)
        finally:
            self.busy = False
            self.current = []
            times = s.engine.profile_stop() if eff["profile"] else None
        dt = time.monotonic() - (state["t_dec0"] or t0)
        total = 0
        for g in gens:
            if g.error is not None:
                raise g.error
            total += len(g.tokens)
            self.out.event("gen", **seq_pairs(g.seq), tokens=len(g.tokens), ms=f"{dt * 1e3:.1f}",
                           tok_per_s=f"{len(g.tokens) / dt if dt > 0 else 0:.2f}", stop=g.stop)
        if multi:
            self.out.event("genall", sequences=nseq, tokens=total, ms=f"{dt * 1e3:.1f}",
                           tok_per_s=f"{total / dt if dt > 0 else 0:.2f}")
        if eff["profile"]:
            for stage in ("prefill", "decode"):        # the reference's fields, src/ops.c:593-603
                self.out.event("profile", stage=stage, **{k: f"{times[stage].get(k, 0.0):.3f}" for k in
                               ("embed", "glue", "qkv", "attn", "wo", "gate_up", "silu", "down", "head", "sample")})
            st = s.engine.manager.stats()
            self.out.event("profile", stage="cache", steps=s.engine.steps_run,
                           pages_high_water=max((g["high_water"] for g in st["groups"]), default=0),
                           pages_reused=sum(g["reused"] for g in st["groups"]))

    def _run_generate(self, s, prompts, eff, eos, on_token, on_prefill):
        """Session.generate, with the scheduler's requests exposed so that SIGINT can cancel them."""
        cli = self
        real_scheduler = s.scheduler

        def watched():
            sch = real_scheduler()
            orig_submit = sch.submit

            def submit(r, forks=()):
                for q in (r, *forks):
                    cli.current.append(q)
                    if cli.cancel:
                        q.cancel = True
                return orig_submit(r, forks=forks)
            sch.submit = submit
            if LEVELS.index(cli.opts["log-level"]) >= LEVELS.index("debug"):
                def on_step(number, plan):           # what each step holds, at the debug level
                    decoded = sum(1 for r, n, _ in plan.entries if n == 1 and r.n_fed > 0)
                    portions = " ".join(f"{r.req_id}:{r.n_fed}+{n}" for r, n, _ in plan.entries if not (n == 1 and r.n_fed > 0))
                    free = min((p.n_free for p in s.engine.manager.pools), default=0)
                    cli.log("debug", f"step={number} tokens={sum(n for _, n, _ in plan.entries)} decoded={decoded} "
                                     f"portions=[{portions}] preempted={len(plan.preempted)} waiting={len(sch.waiting)} "
                                     f"free_pages={free}")
                sch.on_step = on_step
            return sch
        s.scheduler = watched
        try:
            return s.generate(prompts, n=eff["n"], temp=eff["temp"], top_k=eff["top-k"], top_p=eff["top-p"],
                              min_p=eff["min-p"], seed=eff["seed"], max_tokens=eff["max-tokens"],
                              logprobs=eff["logprobs"], timeout=eff["timeout"], eos_ids=eos,
                              on_token=on_token, on_prefill=on_prefill)
        finally:
            s.scheduler = real_scheduler

    def op_bench(self, eff):
        """Prefill and decode speed on seeded random ids, median of --probe-reps runs
        (src/ops.c:942-1030: fresh cache per repetition, prompt in --batch portions, greedy
        decode)."""
        from ..bench_util import bench_once
        s = self.resident(eff)
        reps = []
        for rep in range(eff["probe-reps"]):
            reps.append(bench_once(s, eff["bench-prompt"], eff["bench-gen"], eff["bench-batch"], seed=rep))
        pre = sorted(r[0] for r in reps)[len(reps) // 2]
        dec = sorted(r[1] for r in reps)[len(reps) // 2]
        self.out.event("bench", batch=eff["bench-batch"], prefill_tok_s=f"{pre:.2f}", decode_tok_s=f"{dec:.2f}",
                       prompt_tokens=eff["bench-prompt"], gen_tokens=eff["bench-gen"])

    # ---- one request ------------------------------------------------------------
    def run_request(self, eff):
        """@begin, the operation, @done (src/ops.c:1042-1073). Returns True if it succeeded."""
        t0 = time.monotonic()
        self.requests += 1
        self.cancel = False
        self.out.event("begin", id=eff["id"], op=eff["op"])
        try:
            op = {"generate": self.op_generate, "bench": self.op_bench, "echo": self.op_echo}.get(eff["op"])
            if op is None:
                fail(EINVAL, f"unknown --op '{eff['op']}' (generate, bench, echo)")
            op(eff)
        except EngineError as e:
            self.errors += 1
            self.out.event("done", status="error", code=e.code, msg=e.msg, ms=f"{(time.monotonic() - t0) * 1e3:.1f}")
            return False
        self.out.event("done", status="ok", ms=f"{(time.monotonic() - t0) * 1e3:.1f}")
        return True

    def request_error(self, e):
        self.requests += 1
        self.errors += 1
        self.out.event("begin", id="", op="")
        self.out.event("done", status="error", code=e.code, msg=e.msg, ms="0.0")


def parse_ids(text, vocab):
    """Token ids separated by spaces or commas, each below the vocabulary size (src/ops.c:563-589)."""
    ids = []
    for word in text.replace(",", " ").split():
        if not word.isdigit():
            fail(EINVAL, f"--prompt-ids: '{word}' is not a token id")
        v = int(word)
        if v >= vocab:
            fail(EINVAL, f"--prompt-ids: id {v} is outside the vocabulary of {vocab}")
        ids.append(v)
    if not ids:
        fail(EINVAL, "empty prompt")
    return ids


def effective(session_opts, words):
    eff = dict(session_opts)
    O.apply(eff, words, request=True)
    return eff


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if "--help" in argv or "-h" in argv:
        print("usage: hfamd [options] < requests\n" + O.usage())
        return 0
    try:
        so = O.defaults()
        pre = O.apply(O.defaults(), argv)                   # find --settings first
        if pre["settings"]:
            O.load_settings(so, pre["settings"])
        O.apply(so, argv)
    except EngineError as e:
        print(f"hfamd: {e.msg}", file=sys.stderr)
        return 2
    out = Out(sys.stdout)
    cli = Cli(so, out)
    stop = {"signal": False}

    def on_sigint(signum, frame):                           # src/main.c:19-37
        if cli.busy:
            cli.cancel = True
            for r in cli.current:
                r.cancel = True
        else:
            stop["signal"] = True
            raise KeyboardInterrupt

    def on_sigterm(signum, frame):
        stop["signal"] = True
        raise KeyboardInterrupt
    signal.signal(signal.SIGINT, on_sigint)
    signal.signal(signal.SIGTERM, on_sigterm)
    try:
        signal.signal(signal.SIGPIPE, signal.SIG_IGN)
    except (AttributeError, ValueError):
        pass
    ok = True
    try:
        mode = so["stdin-mode"]
        if mode == "none":
            ok = cli.run_request(dict(so))
        elif mode == "args":
            for raw in sys.stdin:
                if out.err:
                    break
                if len(raw) > so["max-record"]:
                    from ..status import ERANGE
                    cli.request_error(EngineError(ERANGE, "line exceeds --max-record"))
                    continue
                line = raw.strip()
                if not line or line.startswith("#"):
                    continue
                if line.startswith("!"):                     # src/main.c:127-143
                    if line == "!quit":
                        break
                    if line == "!stats":
                        out.event("stats", requests=cli.requests, errors=cli.errors,
                                  live_requests=len(cli.session.engine.manager.held) if cli.session else 0)
                    elif line == "!cancel":
                        out.event("cancel", running=0)
                    else:
                        out.event("error", msg=f"unknown control line '{line}'")
                    continue
                try:
                    eff = effective(so, O.shell_split(line))
                except EngineError as e:
                    cli.request_error(e)
                    continue
                cli.run_request(eff)
        else:
            reader = Reader(sys.stdin.buffer, so["record-sep"], so["max-record"])
            while not out.err:
                try:
                    rec = reader.next()
                except EngineError as e:
                    cli.request_error(e)
                    out.raw(chr(so["record-sep"]))
                    continue
                if rec is None:
                    break
                head, us, body = rec.partition(b"\x1f")       # optional option line before the prompt
                if not us:
                    head, body = b"", rec
                try:
                    eff = effective(so, O.shell_split(head.decode("utf-8", "replace")))
                    text = body.decode("utf-8", "replace").strip()
                    if text:
                        if eff["prompt-ids"] is not None:
                            fail(EINVAL, "--prompt-ids cannot be combined with a prompt record")
                        eff["prompt-ids"] = text                # no tokenizer: the record holds token ids
                    cli.run_request(eff)
                except EngineError as e:
                    cli.request_error(e)
                out.raw(chr(so["record-sep"]))
    except KeyboardInterrupt:
        return 130
    if stop["signal"]:
        return 130
    if out.err:
        return 1
    return 0 if (ok or so["stdin-mode"] != "none") else 1


if __name__ == "__main__":
    sys.exit(main())

"""The programming entry point: one resident model, its engine and scheduler.

The reference's entry points are ``hfc_model_load`` / ``hfc_ctx_new`` /
``hfc_ctx_forward`` (src/model.h:49-79) under a session that keeps one model loaded
between requests (src/ops.h:10-21, src/ops.c:532-561). ``Session`` is that session;
its arguments carry the reference's option names and meanings (``ctx_max``, ``batch``,
``temp``, ``top_k``, ``top_p``, ``min_p``, ``seed``, ``max_tokens``, ``logprobs``,
``n``, ``timeout``; src/opts.c:30-76), and ``engine.step`` is the forward call.
"""
import os
from dataclasses import dataclass, field

import torch

from .engine import Engine
from .engine.scheduler import Request, Scheduler
from .kernels import Ops
from .model import Model, compute_dtype
from .parts.base import FixedState, PagedKV
from .sampling import Sampler, SamplerParams
from .status import EINVAL, ENOMEM, fail


@dataclass
class Generation:
    """One finished sequence."""
    seq: int
    prompt_tokens: int
    tokens: list
    stop: str                          # eos | length | ctx | cancel | timeout, None on error
    logprobs: list = field(default_factory=list)      # per token, if asked for
    top: list = field(default_factory=list)           # per token [(id, logprob), ...], if asked for
    error: object = None
    prefill_s: float = 0.0
    total_s: float = 0.0
    preemptions: int = 0


def cache_bytes_per_token(model):
    """Bytes of paged cache one token takes over all schedule entries."""
    elem = 4 if model.dtype == torch.float32 else 2
    return sum((n.k_width + n.v_width) * elem for n in model.cache_needs() if isinstance(n, PagedKV))


def state_bytes_per_request(model):
    """Bytes of fixed-size state one request holds over all schedule entries (fp32)."""
    return sum(4 * n.n_floats for n in model.cache_needs() if isinstance(n, FixedState))


class Session:
    def __init__(self, model, dtype="bfloat16", ctx_max=32768, batch=64, page_size=16, max_seqs=64,
                 kv_tokens=None, device="cuda:0", seed=0, model_options=None):
        """``model``: a folder with config.json and model.safetensors, or a typed
        configuration (random weights from ``seed`` are then made on the device).
        ``ctx_max``: most tokens per request. ``batch``: tokens per step. ``kv_tokens``:
        tokens the page pools hold (default: ``ctx_max * max_seqs``, but no more than
        most of the free memory allows). ``model_options``: options that change the folder's
        configuration in the engine's own words, e.g. ``{"window": 4096}`` (``--window``); the architecture's
        configuration class turns them into its config.json keys."""
        self.ops = Ops(compute_dtype(dtype), device)
        if isinstance(model, (str, os.PathLike)):
            self.model_dir = os.fspath(model)
            stat = os.stat(os.path.join(self.model_dir, "config.json"))
            self.identity = (os.path.abspath(self.model_dir), stat.st_size, stat.st_mtime)     # src/ops.c:538-545
            self.model = Model.from_dir(self.model_dir, dtype, self.ops, model_options)
        else:
            self.model_dir, self.identity = None, ("random", id(model), seed)
            self.model = Model.from_random(model, seed, dtype, self.ops)
        per_token = cache_bytes_per_token(self.model)
        free, _ = torch.cuda.mem_get_info(self.ops.device)
        free = int(free * 0.8) - (int(max_seqs) + 1) * state_bytes_per_request(self.model)
        if free < 0:
            fail(ENOMEM, f"no memory for the state of {max_seqs} requests "
                         f"({state_bytes_per_request(self.model)} bytes each)")
        if kv_tokens is None:
            kv_tokens = int(ctx_max) * int(max_seqs)
            if per_token:
                kv_tokens = min(kv_tokens, free // per_token)
        ctx_max = int(min(ctx_max, kv_tokens))
        if kv_tokens < page_size:
            fail(ENOMEM, f"no memory for a cache of even one page ({per_token} bytes per token)")
        self.ctx_max, self.batch = ctx_max, int(batch)
        self.engine = Engine(self.model, self.ops, page_tokens=page_size, max_tokens=kv_tokens,
                             max_seqs=max_seqs, max_context=ctx_max)
        self.sampler = Sampler(self.ops)
        self.requests_served = 0

    @property
    def eos_ids(self):
        return tuple(self.model.plan.eos_token_ids)

    def scheduler(self):
        return Scheduler(self.engine, self.sampler, token_budget=self.batch, ctx_max=self.ctx_max)

    def generate(self, prompt_ids, n=1, temp=0.8, top_k=40, top_p=0.95, min_p=0.05, seed=0, max_tokens=512,
                 logprobs=0, timeout=0.0, eos_ids=None, on_token=None, on_prefill=None, on_finish=None):
        """Generates for one prompt (a list of token ids) or several (a list of lists), ``n``
        continuations each; sequence ``i`` of a prompt samples with ``seed + i``
        (src/ops.c:819). All sequences are decoded together. Returns a list of Generation
        in the order (prompt, continuation). The callbacks get (seq, ...) as the scheduler
        produces events."""
        prompts = [prompt_ids] if prompt_ids and isinstance(prompt_ids[0], int) else list(prompt_ids)
        if not prompts:
            fail(EINVAL, "the prompt is empty")
        if not 1 <= n <= 64:
            fail(EINVAL, f"--n {n} is outside 1..64")                               # src/opts.c:54
        params = SamplerParams(float(temp), int(top_k), float(top_p), float(min_p)).check()
        sched = self.scheduler()
        eos = self.eos_ids if eos_ids is None else tuple(eos_ids)
        reqs, families = [], []
        for p in prompts:
            family = [Request(len(reqs) + i, list(p), params, int(max_tokens), int(seed) + i,
                              min(int(logprobs), 64), eos, float(timeout)) for i in range(n)]
            reqs += family
            families.append(family)
        if on_token:
            sched.on_token = lambda r, ch: on_token(r.req_id, len(r.generated) - 1, ch)
        if on_prefill:
            sched.on_prefill = lambda r: on_prefill(r.req_id, r)
        if on_finish:
            sched.on_finish = lambda r: on_finish(r.req_id, r)
        try:
            for family in families:            # the prompt is computed once, the others fork from it
                sched.submit(family[0], forks=family[1:])
            sched.run()
        finally:
            for r in reqs:                     # an error mid-way leaves nothing behind (src/ops.c:930)
                if self.engine.has(r.req_id):
                    self.engine.release(r.req_id)
        self.requests_served += 1
        out = []
        for r in reqs:
            out.append(Generation(r.req_id, len(r.prompt), list(r.generated), r.stop,
                                  [c.logprob for c in r.choices] if r.logprobs else [],
                                  [c.top for c in r.choices] if r.logprobs else [], r.error,
                                  (r.t_first or r.t_done or r.t_submit) - r.t_submit,
                                  (r.t_done or r.t_submit) - r.t_submit, r.preemptions))
        return out


def generate(model, prompt_ids, dtype="bfloat16", **options):
    """One call: load ``model`` (a folder), generate, return the list of Generation.
    Session options (ctx_max, batch, page_size, max_seqs, kv_tokens) and request options
    (n, temp, top_k, top_p, min_p, seed, max_tokens, logprobs, timeout) may be mixed."""
    session_keys = ("ctx_max", "batch", "page_size", "max_seqs", "kv_tokens", "device")
    s_opts = {k: options.pop(k) for k in session_keys if k in options}
    return Session(model, dtype=dtype, **s_opts).generate(prompt_ids, **options)

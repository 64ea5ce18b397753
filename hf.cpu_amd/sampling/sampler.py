"""Sampling the next token from a row of logits.

The pipeline and its order are the reference's ``hfc_sample`` (src/sample.c:66-117):
greedy when the temperature is not positive (first index of the maximum); otherwise
candidates ordered by (logit descending, id ascending), cut to ``top_k``, turned into
probabilities ``exp((l - max) / temp)`` normalised in fp32, cut by ``min_p`` (leading run
with ``p >= min_p * p_max``), cut by ``top_p`` (shortest prefix whose sum reaches it), and
one draw ``r = uniform * sum`` picks the first candidate whose running sum exceeds ``r``.

The GPU does all of it (kernels in csrc/sampling.hip): argmax; the ordered best-k and the
row's log-sum-exp, or, with ``top_k`` off (0) or beyond the best-k kernel's 1024, the whole
row in order; and the draw from these candidates, with every operation rounded to fp32 and nothing
fused, in the reference's order. The host gives each request's uniform number and reads one
token a row.
"""
from dataclasses import dataclass

import numpy as np
import torch

from .. import memory
from ..status import EINVAL, fail

TOPK_KERNEL_MAX = 1024
f32 = np.float32


@dataclass(frozen=True)
class SamplerParams:
    """Defaults are the reference's (src/opts.c:102-106)."""
    temp: float = 0.8
    top_k: int = 40
    top_p: float = 0.95
    min_p: float = 0.05

    def check(self):
        if not 0 <= self.temp <= 5:
            fail(EINVAL, f"--temp {self.temp} is outside 0..5")                 # src/opts.c:55
        if not 0 <= self.top_k <= 1000000:
            fail(EINVAL, f"--top-k {self.top_k} is outside 0..1000000")
        if not 0 <= self.top_p <= 1 or not 0 <= self.min_p <= 1:
            fail(EINVAL, "--top-p and --min-p must lie in 0..1")
        return self

    @property
    def greedy(self):
        return self.temp <= 0


@dataclass
class Choice:
    token: int
    logprob: float = None          # of the chosen token, if asked for
    top: list = None               # [(id, logprob), ...] best first, if asked for


class Started:
    """A step's sampling under way (``Sampler.sample_start``)."""

    def __init__(self, device_tokens, choices, read=None):
        self.device_tokens, self._choices, self._read = device_tokens, choices, read

    def finish(self):
        if self._choices is None:
            self._choices = self._read()
        return self._choices


class Sampler:
    """Samples one token per row of a step's logits. ``wants[i]`` = (params, rng, n_logprobs)."""

    def __init__(self, ops):
        self.ops = ops
        self._landing = []            # pinned host buffers that chosen tokens are copied to, used in turn
        self._turn = 0
        self._outbox = []             # pinned host buffers that the draws' numbers leave from: [tensor, event of its last copy]
        self._out_turn = 0

    def _to_host_later(self, tokens):
        """Enqueues the copy of ``tokens`` (int32 on the device) to pinned host memory right behind the
        kernel that writes them, and returns a function that waits for that copy alone and gives the
        numbers: a plain read would wait for everything enqueued since, the next step included."""
        n = tokens.numel()
        if len(self._landing) < 4:
            self._landing.append(memory.empty(max(n, 256), torch.int32, None, "pinned buffer for chosen tokens", pin=True))
        self._turn = (self._turn + 1) % len(self._landing)
        if self._landing[self._turn].numel() < n:
            self._landing[self._turn] = memory.empty(2 * n, torch.int32, None, "pinned buffer for chosen tokens", pin=True)
        host = self._landing[self._turn][:n]
        host.copy_(tokens, non_blocking=True)
        done = torch.cuda.Event()
        done.record()

        def read():
            done.synchronize()
            return host.numpy().copy()
        return read

    def _draw(self, ids, vals, numbers, cuts, on_device=False):
        """The device's draw for rows of candidates in order; the rows' numbers and cuts travel as one copy."""
        n = len(cuts)
        sent = self._send(numbers, cuts, vals.device)
        drawn = self.ops.draw_rows(ids, vals, sent[:4 * n].view(n, 4), sent[4 * n:].view(torch.int32))
        return drawn if on_device else drawn.cpu().numpy()

    def _send(self, numbers, cuts, device):
        """The rows' numbers ([n, 4] fp32) and cuts ([n] int32) on the device as one fp32 tensor of 5 n, by a
        copy from pinned memory that only enqueues: a copy from pageable memory makes the host wait for
        everything the stream holds, the step that was just enqueued included. Four host buffers take turns;
        one is written again only after the copy that last read it is done."""
        n = len(cuts)
        if len(self._outbox) < 4:
            self._outbox.append([memory.empty(max(5 * n, 1280), torch.float32, None, "pinned buffer for the draws' numbers", pin=True), None])
        self._out_turn = (self._out_turn + 1) % len(self._outbox)
        box = self._outbox[self._out_turn]
        if box[1] is not None:
            box[1].synchronize()
        if box[0].numel() < 5 * n:
            box[0] = memory.empty(10 * n, torch.float32, None, "pinned buffer for the draws' numbers", pin=True)
        flat = box[0].numpy()
        flat[:4 * n] = np.asarray(numbers, dtype=f32).reshape(-1)
        flat[4 * n:5 * n].view(np.int32)[:] = cuts
        sent = memory.empty(5 * n, torch.float32, device, "the draws' numbers")
        sent.copy_(box[0][:5 * n], non_blocking=True)
        box[1] = torch.cuda.Event()
        box[1].record()
        return sent

    def sample_start(self, logits, wants):
        """Begins the sampling of a step's rows and returns a ``Started``: ``device_tokens`` is the int32
        tensor of the chosen tokens on the device if they can be had without the host (all rows greedy, or
        all rows drawn from their best k, none asking for log-probabilities), else None; ``finish()``
        returns the list of Choice (and waits for the device). Between the two the caller may enqueue
        the next step with ``device_tokens`` as its input: ``logits`` is not read after this call returns
        unless ``device_tokens`` is None, in which case everything has been computed already. Each
        request's generator moves on here, by one draw, as in ``sample``."""
        R, V = logits.shape
        if R != len(wants):
            fail(EINVAL, f"sampler: {R} rows of logits for {len(wants)} requests")
        if any(n_lp for _, _, n_lp in wants):
            return Started(None, self.sample(logits, wants))
        if all(p.greedy for p, _, _ in wants):
            arg = self.ops.argmax(logits)
            read = self._to_host_later(arg)
            return Started(arg, None, lambda: [Choice(int(t)) for t in read()])
        if all(not p.greedy and 0 < p.top_k <= TOPK_KERNEL_MAX and p.top_k < V for p, _, _ in wants):
            k = max(p.top_k for p, _, _ in wants)
            ids, vals, _ = self.ops.topk(logits, k, want_stats=False)
            numbers = np.array([(p.temp, p.top_p, p.min_p, rng.uniform()) for p, rng, _ in wants], dtype=f32)
            cuts = np.array([p.top_k for p, _, _ in wants], dtype=np.int32)
            drawn = self._draw(ids, vals, numbers, cuts, on_device=True)
            read = self._to_host_later(drawn)
            return Started(drawn, None, lambda: [Choice(int(t)) for t in read()])
        return Started(None, self.sample(logits, wants))

    def sample(self, logits, wants):
        R = logits.shape[0]
        if R != len(wants):
            fail(EINVAL, f"sampler: {R} rows of logits for {len(wants)} requests")
        out = [None] * R
        need_k = 0
        for params, _, n_lp in wants:
            if n_lp or (not params.greedy and 0 < params.top_k <= TOPK_KERNEL_MAX):
                need_k = max(need_k, n_lp, 0 if params.greedy else min(params.top_k, TOPK_KERNEL_MAX))
        need_k = min(need_k, logits.shape[1])
        V = logits.shape[1]
        greedy = [i for i, (p, _, _) in enumerate(wants) if p.greedy]
        arg = self.ops.argmax(logits).cpu().numpy() if greedy else None
        best = ids = vals = stats = None
        if need_k or any(n for _, _, n in wants):
            best = self.ops.topk(logits, need_k)
            if any(n for _, _, n in wants):       # before the draw below turns the values into probabilities
                ids, vals, stats = (t.cpu().numpy() for t in best)
        toks = [None] * R
        few = []                                  # rows drawn from the best-k kernel's candidates
        whole = []                                # rows drawn from the whole vocabulary, in order
        for i, (params, rng, n_lp) in enumerate(wants):
            if params.greedy:
                toks[i] = int(arg[i])
            elif 0 < params.top_k <= TOPK_KERNEL_MAX and params.top_k < V:
                few.append(i)
            else:
                whole.append(i)
        # Either way the device draws (csrc/sampling.hip); the host gives each request's uniform number and
        # reads back one token a row.
        if few:
            numbers = np.zeros((R, 4), dtype=f32)
            numbers[:, :2] = 1                    # rows that are not drawn here: any harmless draw
            cuts = np.ones(R, dtype=np.int32)
            for i in few:
                params, rng, _ = wants[i]
                numbers[i] = (params.temp, params.top_p, params.min_p, rng.uniform())
                cuts[i] = params.top_k
            drawn = self._draw(best[0], best[1], numbers, cuts)
            for i in few:
                toks[i] = int(drawn[i])
        if whole:
            chosen = None if len(whole) == R else memory.to_device(torch.tensor(whole, dtype=torch.int32), logits.device, "rows to order")
            all_ids, all_vals = self.ops.order_rows(logits, chosen)
            numbers = np.empty((len(whole), 4), dtype=f32)
            cuts = np.empty(len(whole), dtype=np.int32)
            for j, i in enumerate(whole):
                params, rng, _ = wants[i]
                numbers[j] = (params.temp, params.top_p, params.min_p, rng.uniform())
                cuts[j] = params.top_k if 0 < params.top_k < V else V
            for i, t in zip(whole, self._draw(all_ids, all_vals, numbers, cuts)):
                toks[i] = int(t)
        for i, (params, rng, n_lp) in enumerate(wants):
            tok = toks[i]
            ch = Choice(tok)
            if n_lp:
                mx, lse = float(stats[i, 0]), float(stats[i, 1])
                ch.top = [(int(t), float(v) - mx - lse) for t, v in zip(ids[i, :n_lp], vals[i, :n_lp])]
                hit = [lp for t, lp in ch.top if t == tok]
                ch.logprob = hit[0] if hit else float(logits[i, tok].item()) - mx - lse     # src/sample.c:25-33
            out[i] = ch
        return out

"""Timing a prefill and a run of decode steps through the scheduler's own path.

Shared by ``--op bench`` and the repository's bench.py. Prompts are seeded pseudo-random
ids below min(vocab, 2000), as in the reference's bench op (src/ops.c:977-979).
"""
import time

import numpy as np
import torch


def random_prompts(vocab, n_prompts, length, seed):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, min(vocab, 2000), length)] for _ in range(n_prompts)]


def bench_once(session, n_prompt, n_gen, n_seqs, seed=0):
    """(prefill tokens/s, decode tokens/s) for ``n_seqs`` prompts of ``n_prompt`` ids and
    ``n_gen`` greedy tokens each, on a cache that starts empty."""
    eng, ops = session.engine, session.ops
    prompts = random_prompts(session.model.vocab_size, n_seqs, n_prompt, seed)
    budget = session.batch
    ids = list(range(n_seqs))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    last = {}
    for i in ids:
        at = 0
        while at < n_prompt:
            n = min(budget, n_prompt - at)
            final = at + n == n_prompt
            logits = eng.step([(("bench", i), prompts[i][at:at + n], [n - 1] if final else [])])
            at += n
        last[i] = int(ops.argmax(logits).cpu()[0])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    # as the scheduler decodes: a step takes its tokens from the device, the host reads them a step late
    dev = torch.tensor([last[i] for i in ids], dtype=torch.int32, device=ops.device)
    rows = {i: i for i in range(n_seqs)}
    read = None
    for _ in range(n_gen):
        logits = eng.step([(("bench", i), [0], [0]) for i in ids], fed=(dev, rows))
        dev = ops.argmax(logits)
        if read is not None:
            read()
        read = session.sampler._to_host_later(dev)
    read()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    for i in ids:
        eng.release(("bench", i))
    return n_seqs * n_prompt / (t1 - t0), n_seqs * n_gen / (t2 - t1)

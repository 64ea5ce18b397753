"""The sampler's draw written out in numpy for whole arrays of rows: a quick stand-in for the plain,
scalar sampler of tests/plain.py where that one is too slow (rows of 152,064 candidates), itself
pinned to it by tests/test_sampling_cli.py. Nothing of the package is used here.

``hfc_expf``: the reference's exponential (src/mathx.c:7-32), operation for operation in fp32: the
sampler's probabilities are exp((l - max) / temp) by this routine, not by a library's exp; a draw
compares a running fp32 sum with a threshold, so one unit in the last place of one probability can
move it to another token.
"""
import numpy as np

f32 = np.float32


def hfc_expf(x):
    """exp(x) for an fp32 array: 2^n * exp(r) with r = x - n ln2 in two steps and a degree-7
    polynomial, every operation rounded to fp32 (src/mathx.c:15-31)."""
    x0 = np.asarray(x, dtype=f32)
    with np.errstate(invalid="ignore", over="ignore"):
        x = np.minimum(x0, f32(88.3762626647949))
        fx = np.floor(x * f32(1.44269504088896341) + f32(0.5))
        n = np.nan_to_num(fx, nan=0.0).astype(np.int32)
        x = x - fx * f32(0.693359375)
        x = x - fx * f32(-2.12194440e-4)
        z = x * x
        y = f32(1.9875691500e-4)
        y = y * x + f32(1.3981999507e-3)
        y = y * x + f32(8.3334519073e-3)
        y = y * x + f32(4.1665795894e-2)
        y = y * x + f32(1.6666665459e-1)
        y = y * x + f32(5.0000001201e-1)
        y = y * z + x + f32(1.0)
        p2 = ((np.clip(n, -126, 128) + 127).astype(np.uint32) << np.uint32(23)).view(f32)
        out = (y * p2).astype(f32)
    out = np.where(x0 < f32(-87.3365478515625), f32(0.0), out)
    return np.where(np.isnan(x0), x0, out).astype(f32)


def pick_rows(ids, logits, params, rngs):
    """The draw for several rows with the same parameters: ``ids`` and ``logits`` are [R, k]
    candidates already ordered (logit descending, id ascending) and cut to top_k; ``rngs[r]``
    is row r's generator. Steps 3 to 6 of the pipeline in fp32 (src/sample.c:99-114): every
    sum is a running fp32 sum in candidate order, as in the reference's loops (``cumsum``
    adds one element at a time in the array's precision)."""
    logits = np.asarray(logits, dtype=f32)
    ids = np.asarray(ids)
    R, k = logits.shape
    col = np.arange(k)[None, :]
    p = hfc_expf((logits - logits[:, :1]) / f32(params.temp))               # src/sample.c:99, src/mathx.c:7-32
    p = (p / np.cumsum(p, axis=1, dtype=f32)[:, -1:]).astype(f32)
    kept = np.full(R, k)
    if params.min_p > 0:
        below = p < f32(params.min_p) * p[:, :1]                 # p does not increase along the order
        kept = np.maximum(np.where(below.any(axis=1), below.argmax(axis=1), k), 1)
    if 0 < params.top_p < 1:
        live = col < kept[:, None]
        reached = (np.cumsum(np.where(live, p, f32(0)), axis=1, dtype=f32) >= f32(params.top_p)) & live
        kept = np.where(reached.any(axis=1), reached.argmax(axis=1) + 1, kept)
    live = col < kept[:, None]
    cum = np.cumsum(np.where(live, p, f32(0)), axis=1, dtype=f32)
    u = np.array([rng.uniform() for rng in rngs], dtype=f32)     # 24 random bits: exact in fp32
    r = u * cum[np.arange(R), kept - 1]
    over = (r[:, None] < cum) & live
    at = np.where(over.any(axis=1), over.argmax(axis=1), kept - 1)
    return [int(t) for t in ids[np.arange(R), at]]


def pick(ids, logits, params, rng):
    """One row of ``pick_rows``."""
    return pick_rows(np.asarray(ids)[None, :], np.asarray(logits, dtype=f32)[None, :], params, [rng])[0]


def order_on_host(row, top_k):
    """All candidates of a row in order, cut to top_k if it is on (src/sample.c:59-64, 81-98): the
    order that the device's kernels give, written out in numpy for the tests of ``pick``."""
    row = np.asarray(row, dtype=f32)
    order = np.argsort(-row, kind="stable")                 # logit descending, ties by id ascending
    if 0 < top_k < len(order):
        order = order[:top_k]
    return order.astype(np.int64), row[order]

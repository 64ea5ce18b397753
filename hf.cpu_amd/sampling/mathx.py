"""The reference's exponential (src/mathx.c:7-32), operation for operation in fp32.

The sampler's probabilities are exp((l - max) / temp) by this routine, not by a library's
exp: a draw compares a running fp32 sum with a threshold, so one unit in the last place of one
probability can move it to another token. The same sequence of fp32 operations (no fused
multiply-add) is what the device's draw kernel runs.
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

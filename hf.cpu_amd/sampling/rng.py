"""The sampler's random numbers: xorshift64*, bit for bit the reference's
(src/sample.c:9-23), so that a seed means the same sequence of draws."""
import numpy as np

MASK64 = (1 << 64) - 1


class Rng:
    def __init__(self, seed):
        self.s = (int(seed) * 0x9e3779b97f4a7c15 + 0x1234567) & MASK64
        if self.s == 0:
            self.s = 0x2545f4914f6cdd1d

    def next_u64(self):
        x = self.s
        x ^= x >> 12
        x ^= (x << 25) & MASK64
        x ^= x >> 27
        self.s = x
        return (x * 0x2545f4914f6cdd1d) & MASK64

    def uniform(self):
        """A float32 in [0, 1) with 24 random bits."""
        return np.float32(self.next_u64() >> 40) / np.float32(16777216.0)

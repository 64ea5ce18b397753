"""The device's own peaks, measured: what a streaming read, a copy and a burn of the matrix cores
reach on this GPU (the reference measures its machine the same way with ``read_sum`` and
``fma_burn``, src/kern.h:17-23, src/probe.c). The bench prices its kernels against these beside the
published figures."""
import ctypes

import torch

from .status import EINVAL, EngineError
from .kernels.lib import last_error


def _timed(fn, reps):
    """Median milliseconds of ``reps`` runs of ``fn`` after one warm-up, by device events."""
    fn()
    times = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b))
    return sorted(times)[len(times) // 2]


def measure_peaks(ops, read_bytes=2 << 30, reps=5, mfma_iters=1 << 15):
    """{"hbm_read_GBps", "hbm_copy_GBps", "mfma_bf16_TFLOPs", "mfma_bf16_zero_TFLOPs"}: a
    flat read of ``read_bytes`` (far more than the caches hold), a copy of half as much (bytes read plus
    bytes written count), and the matrix cores on random and on all-zero register operands."""
    lib = ops.lib
    stream = lambda: torch.cuda.current_stream(ops.device).cuda_stream

    def check(rc):
        if rc:
            raise EngineError(EINVAL, last_error())

    buf = torch.empty(read_bytes, dtype=torch.uint8, device=ops.device)
    buf.random_(0, 255)
    sink = torch.zeros(16, dtype=torch.uint8, device=ops.device)
    out = {}
    best = 0.0
    for per_cu in (4, 8, 16, 32):          # the best of a few launch shapes is what the device can do
        ms = _timed(lambda: check(lib.hfa_probe_read(buf.data_ptr(), read_bytes, sink.data_ptr(), per_cu, stream())), reps)
        best = max(best, read_bytes / ms / 1e6)
    out["hbm_read_GBps"] = round(best, 1)
    half = read_bytes // 2
    ms = _timed(lambda: check(lib.hfa_probe_copy(buf.data_ptr(), buf.data_ptr() + half, half, stream())), reps)
    out["hbm_copy_GBps"] = round(2 * half / ms / 1e6, 1)
    del buf
    acc = torch.empty(int(lib.hfa_probe_mfma_threads()), dtype=torch.float32, device=ops.device)
    flops = ctypes.c_double(0.0)
    for key, zeros in (("mfma_bf16_TFLOPs", 0), ("mfma_bf16_zero_TFLOPs", 1)):
        ms = _timed(lambda: check(lib.hfa_probe_mfma(acc.data_ptr(), mfma_iters, zeros, ctypes.byref(flops), stream())), reps)
        out[key] = round(flops.value / ms / 1e9, 1)
    return out

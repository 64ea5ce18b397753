"""The one place where the engine asks for device memory (and pinned host memory).

Every tensor the engine allocates itself (weights, cache storage, work buffers, staging
buffers, the sampler's outputs) and every graph it captures passes through here, so
that allocations can be counted and, for tests, made to fail: the reference's checked
allocator with fault injection (``hfc_fail_after`` and the environment variable
``HFC_FAIL_AFTER``, src/mem.c:12-30), swept by its tests (tests/e2e.pl:175-179). A
failed allocation, injected or real, is ``EngineError(ENOMEM)``; whoever holds
half-built state gives it back on the way up.

``HFAMD_FAIL_AFTER=n`` in the environment (read at the first allocation) or
``fail_after(n)`` makes the n-th allocation from then on fail, once.
"""
import os

import torch

from .status import ENOMEM, EngineError

_fail_after = None           # None: the environment has not been read yet
_count = 0


def fail_after(n):
    """The n-th allocation from now fails (0: none does)."""
    global _fail_after
    _fail_after = max(int(n), 0)


def allocations():
    """How many allocations were asked for so far."""
    return _count


def note(what):
    """Counts one allocation named ``what`` that is about to happen elsewhere (a library call
    that allocates: a concatenation, a graph capture); raises if it is the one to fail."""
    global _fail_after, _count
    if _fail_after is None:
        try:
            _fail_after = max(int(os.environ.get("HFAMD_FAIL_AFTER", "0") or 0), 0)
        except ValueError:
            _fail_after = 0
    _count += 1
    if _fail_after > 0:
        _fail_after -= 1
        if _fail_after == 0:
            raise EngineError(ENOMEM, f"allocation {_count} ({what}) failed (injected failure)")


def _real(what, fn):
    note(what)
    try:
        return fn()
    except torch.cuda.OutOfMemoryError as e:
        raise EngineError(ENOMEM, f"out of device memory for {what}: {str(e).splitlines()[0]}") from None


def empty(shape, dtype, device, what, pin=False):
    if pin:
        return _real(what, lambda: torch.empty(shape, dtype=dtype, pin_memory=True))
    return _real(what, lambda: torch.empty(shape, dtype=dtype, device=device))


def zeros(shape, dtype, device, what):
    return _real(what, lambda: torch.zeros(shape, dtype=dtype, device=device))


def to_device(tensor, device, what, dtype=None):
    """``tensor`` (host or device) on ``device`` in ``dtype``, contiguous."""
    return _real(what, lambda: tensor.to(device=device, dtype=dtype or tensor.dtype).contiguous())


def cat(tensors, dim, what):
    return _real(what, lambda: torch.cat(tensors, dim=dim).contiguous())

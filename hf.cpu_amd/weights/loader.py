"""Loading a model's tensors by name, with one error for everything that is wrong.

Per-tensor checks are the reference's (src/model.c:52-93: missing tensor, wrong
shape, type without a kernel); here they are gathered over the whole file first,
so that one message lists every missing tensor, every unexpected one and every
wrong shape.
"""
import torch

from .. import memory

from ..status import EFORMAT, fail
from .safetensors_io import open_model_tensors

FLOAT_STORED = ("F32", "BF16", "F16")
INT_STORED = ("I64", "I32", "I16", "I8", "U8")
LIST_LIMIT = 12


def _listing(names):
    names = list(names)
    shown = ", ".join(names[:LIST_LIMIT])
    return shown + (f", ... ({len(names)} in all)" if len(names) > LIST_LIMIT else "")


def check_tensors(entries, specs, origin):
    """Raises EFORMAT naming all missing, unexpected, wrongly shaped and wrongly typed tensors."""
    by_name = {s.name: s for s in specs}
    missing = [s.name for s in specs if not s.optional and s.name not in entries]
    unexpected = [n for n in entries if n not in by_name]
    shapes, types = [], []
    for s in specs:
        e = entries.get(s.name)
        if e is None:
            continue
        if tuple(e.shape) != tuple(s.shape):
            shapes.append(f"{s.name} has shape {'x'.join(map(str, e.shape)) or 'scalar'}, "
                          f"expected {'x'.join(map(str, s.shape))}")     # src/model.c:80-82
        allowed = INT_STORED if s.kind == "table" else FLOAT_STORED
        if e.dtype not in allowed:
            types.append(f"{s.name} is stored as {e.dtype} (allowed: {', '.join(allowed)})")   # src/model.c:83-84
    problems = []
    if missing:
        problems.append(f"missing tensors: {_listing(missing)}")
    if unexpected:
        problems.append(f"unexpected tensors: {_listing(unexpected)}")
    if shapes:
        problems.append(f"wrong shapes: {_listing(shapes)}")
    if types:
        problems.append(f"unsupported types: {_listing(types)}")
    if problems:
        fail(EFORMAT, f"{origin}: " + "; ".join(problems))


def held_dtype(kind, stored, compute_dtype):
    """The dtype a tensor is held in on the device. Matrices are held in the compute
    dtype, except that one stored in 32-bit stays in 32-bit; vectors are widened to
    fp32 (exact); integer tables become int32."""
    if kind == "table":
        return torch.int32
    if kind == "vector" or stored == "F32" or compute_dtype == torch.float32:
        return torch.float32
    return compute_dtype


def load_tensors(model_dir, specs, compute_dtype, device):
    """name -> device tensor for every spec found in the folder's safetensors."""
    entries = open_model_tensors(model_dir)
    check_tensors(entries, specs, model_dir)
    out = {}
    for s in specs:
        e = entries.get(s.name)
        if e is None:
            continue
        t = e.file.read(s.name)
        out[s.name] = memory.to_device(t, device, f"tensor '{s.name}'", held_dtype(s.kind, e.dtype, compute_dtype))
    return out

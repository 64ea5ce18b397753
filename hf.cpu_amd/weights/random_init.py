"""Random weights: a model folder written from a configuration and a seed, and the
same numbers made straight in device memory for measurements.

Rules (per tensor, chosen by its ParamSpec): matrices and biases N(0, std), norm scales
1 + N(0, std); integer tables uniform below their bound. The role is that of the reference's
tools/mkmodel.pl:104-127 (one generator for the tiny model and for the oracle that checks it: a
sum of uniform numbers as the Gaussian), so the file and the device hold the same bits:

* The generator is a counter, not a stream: tensor ``i`` of the plan (in the order of its tensor
  declarations) has the key ``mix(seed * 0x9e3779b97f4a7c15 + i)``, and element ``e`` (row-major)
  takes the two 64-bit words ``mix(key + 2e)`` and ``mix(key + 2e + 1)``, with ``mix`` the
  finishing function of splitmix64 (``z ^= z >> 30; z *= 0xbf58476d1ce4e5b9; z ^= z >> 27;
  z *= 0x94d049bb133111eb; z ^= z >> 31``, all modulo 2^64). A tensor's values do not depend on
  which other tensors are made, nor on where or in which order its elements are computed.
* The eight 16-bit fields of the two words are added up: ``S`` in 0..524280, mean 262140,
  variance 8 (65536^2 - 1) / 12. The value is ``fp32(S - 262140) * fp32(std / sqrt(variance))``:
  an exact integer and one fp32 product, the same on any machine; ``1 +`` it for norm scales
  (one fp32 sum); then rounded to the stored dtype (nearest even). The sum of eight uniform
  numbers is Gaussian to within what a random test model needs (no value beyond 4.9 std).
* A table takes ``mix(key + 2e)`` modulo its bound.

``random_values`` is the statement of the rule in numpy; ``hfa_random_fill`` (csrc/elementwise.hip)
computes the same on the device.
"""
import json
import math
import os

import numpy as np
import torch

from .. import memory
from .safetensors_io import write_safetensors

STORED = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}
MASK64 = (1 << 64) - 1
GOLDEN = 0x9e3779b97f4a7c15
SUM_MEAN = 262140                                            # 8 fields of mean 32767.5
SUM_STD = math.sqrt(8 * (65536.0 ** 2 - 1) / 12)


def _mix_int(z):
    z &= MASK64
    z = ((z ^ (z >> 30)) * 0xbf58476d1ce4e5b9) & MASK64
    z = ((z ^ (z >> 27)) * 0x94d049bb133111eb) & MASK64
    return z ^ (z >> 31)


def tensor_key(seed, index):
    """The key of tensor ``index`` under ``seed`` (a 64-bit integer)."""
    return _mix_int(int(seed) * GOLDEN + int(index))


def unit_scale(std):
    """fp32 factor that turns ``S - 262140`` into N(0, std)."""
    return np.float32(float(std) / SUM_STD)


def _mix(z):
    with np.errstate(over="ignore"):
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xbf58476d1ce4e5b9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94d049bb133111eb)
        return z ^ (z >> np.uint64(31))


def random_values(key, count, rule, param, first=0):
    """Elements ``first .. first + count - 1`` of the tensor with ``key``: fp32 for the rules
    "normal" and "one_plus_normal" (``param`` = std), int32 for "table" (``param`` = bound)."""
    with np.errstate(over="ignore"):
        e = np.arange(first, first + count, dtype=np.uint64)
        a = _mix(np.uint64(key) + np.uint64(2) * e)
        if rule == "table":
            return (a % np.uint64(int(param))).astype(np.int32)
        b = _mix(np.uint64(key) + np.uint64(2) * e + np.uint64(1))
    total = np.zeros(count, dtype=np.int64)
    for word in (a, b):
        for shift in (0, 16, 32, 48):
            total += ((word >> np.uint64(shift)) & np.uint64(0xffff)).astype(np.int64)
    vals = (total - SUM_MEAN).astype(np.float32) * unit_scale(param)
    if rule == "one_plus_normal":
        vals = np.float32(1.0) + vals
    elif rule != "normal":
        raise ValueError(f"unknown init rule '{rule}'")
    return vals.astype(np.float32)


def random_tensor(spec, seed, index, dtype):
    """Tensor ``index`` of the plan on the host, in ``dtype``."""
    count = int(np.prod(spec.shape, dtype=np.int64))
    key = tensor_key(seed, index)
    rule = "table" if spec.kind == "table" else spec.init[0]
    out = np.empty(count, dtype=np.int32 if rule == "table" else np.float32)
    for at in range(0, count, 1 << 22):                      # in pieces: the integers take 8 bytes an element
        n = min(1 << 22, count - at)
        out[at:at + n] = random_values(key, n, rule, spec.init[1], first=at)
    t = torch.from_numpy(out.reshape(spec.shape))
    return t if rule == "table" else t.to(dtype)


def write_random_model(model_dir, config, seed, dtype="float32"):
    """Writes ``config.json`` and ``model.safetensors`` for ``config`` (a typed
    configuration of a registered architecture). Optional tensors (a tied head) are
    not written. Returns the folder."""
    from ..model import Model
    stored = STORED[dtype]
    os.makedirs(model_dir, exist_ok=True)
    obj = config.to_dict()
    obj["torch_dtype"] = dtype
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(obj, f, indent=1)
    specs = [s for s in Model.from_config(config).param_specs() if not s.optional]
    tensors = {}
    for i, s in enumerate(specs):
        dt = torch.int32 if s.kind == "table" else stored
        tensors[s.name] = (dt, tuple(s.shape), (lambda s=s, i=i, dt=dt: random_tensor(s, seed, i, dt)))
    write_safetensors(os.path.join(model_dir, "model.safetensors"), tensors,
                      {"format": "pt", "seed": seed})
    return model_dir


def random_device_tensors(specs, seed, compute_dtype, device, ops=None):
    """The tensors ``write_random_model`` would write with ``seed`` in the held dtype, made on the
    device (``hfa_random_fill``): the same bits as loading that file, without the file; for
    models too large to be worth one."""
    import ctypes
    from ..kernels.lib import last_error, library
    from ..status import EINVAL, EngineError
    from .loader import held_dtype
    lib = library()
    stream = torch.cuda.current_stream(device).cuda_stream
    code = {torch.float32: 0, torch.bfloat16: 1, torch.int32: 2}
    out = {}
    index = 0
    for s in specs:
        if s.optional:
            continue
        key = tensor_key(seed, index)
        index += 1
        rule = "table" if s.kind == "table" else s.init[0]
        if rule not in ("table", "normal", "one_plus_normal"):
            raise ValueError(f"unknown init rule '{rule}' for {s.name}")
        # what the file would hold (the writer's dtype is the compute dtype here), then what the loader keeps
        stored = torch.int32 if rule == "table" else compute_dtype
        held = held_dtype(s.kind, "F32" if compute_dtype == torch.float32 else "BF16", compute_dtype)
        t = memory.empty(s.shape, stored, device, f"tensor '{s.name}'")
        rc = lib.hfa_random_fill(t.data_ptr(), code[stored], ctypes.c_size_t(t.numel()), ctypes.c_uint64(key),
                                 ctypes.c_float(0.0 if rule == "table" else float(unit_scale(s.init[1]))),
                                 {"normal": 0, "one_plus_normal": 1, "table": 2}[rule],
                                 int(s.init[1]) if rule == "table" else 0, stream)
        if rc:
            raise EngineError(EINVAL, last_error())
        out[s.name] = t if held == stored else memory.to_device(t, device, f"tensor '{s.name}' widened", held)
    return out

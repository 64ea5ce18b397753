"""Random weights: a model folder written from a configuration and a seed, and the
same rules applied straight to device memory for measurements.

Rules (per tensor, chosen by its ParamSpec): matrices and biases N(0, std), norm
scales 1 + N(0, std). Tensor ``i`` of the plan draws from numpy's PCG64 seeded with
``(seed, i)``, in fp64 rounded to fp32 and then to the stored dtype, so a tensor's
values do not depend on which other tensors are made. The role is that of the
reference's tools/mkmodel.pl:104-127 (a tiny random model for the oracle test).
"""
import json
import os

import numpy as np
import torch

from .. import memory

from .safetensors_io import write_safetensors

STORED = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def random_tensor(spec, seed, index, dtype):
    rng = np.random.Generator(np.random.PCG64([int(seed), int(index)]))
    count = int(np.prod(spec.shape, dtype=np.int64))
    rule = spec.init[0]
    if spec.kind == "table":
        return torch.from_numpy(rng.integers(0, int(spec.init[1]), size=count, dtype=np.int32).reshape(spec.shape))
    vals = rng.standard_normal(count, dtype=np.float64) * float(spec.init[1])
    if rule == "one_plus_normal":
        vals += 1.0
    elif rule != "normal":
        raise ValueError(f"unknown init rule '{rule}' for {spec.name}")
    return torch.from_numpy(vals.astype(np.float32).reshape(spec.shape)).to(dtype)


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


def random_device_tensors(specs, seed, compute_dtype, device):
    """The same rules drawn by the device's generator (another stream of numbers than
    the file writer's): for models too large to be worth a file."""
    from .loader import held_dtype
    gen = torch.Generator(device=device)
    out = {}
    for i, s in enumerate(specs):
        if s.optional:
            continue
        gen.manual_seed(int(seed) * 1000003 + i)
        held = held_dtype(s.kind, "BF16", compute_dtype)
        if s.kind == "table":
            out[s.name] = torch.randint(0, int(s.init[1]), s.shape, generator=gen, device=device, dtype=torch.int32)
            continue
        t = memory.empty(s.shape, held, device, f"tensor '{s.name}'")
        t.normal_(0.0, float(s.init[1]), generator=gen)
        if s.init[0] == "one_plus_normal":
            t += 1.0
        out[s.name] = t
    return out

"""A model: the parts a plan names, built, with their tensors bound.

``Model.from_dir`` is the one way in for a model folder: config.json names the
architecture, the registry gives its configuration class and plan function, the
plan gives the parts, the parts declare the tensors the loader must find.
"""
import torch

from .config import config_from_dict, read_config
from .parts.base import FixedState, PagedKV
from .parts.block import norm_for
from .registry import architecture, make_part
from .status import EINVAL, fail
from .weights.loader import load_tensors
from .weights.random_init import random_device_tensors

COMPUTE_DTYPES = {"float32": torch.float32, "fp32": torch.float32,
                  "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def compute_dtype(name):
    if isinstance(name, torch.dtype):
        return name
    if name not in COMPUTE_DTYPES:
        fail(EINVAL, f"dtype '{name}' is not one of {', '.join(sorted(COMPUTE_DTYPES))}")
    return COMPUTE_DTYPES[name]


class Layer:
    """A layer's block and the parts it arranges, by the names the plan gave them (also as attributes)."""

    def __init__(self, label, block, named):
        self.label, self.block, self.named = label, block, dict(named)
        for name, part in self.named.items():
            setattr(self, name, part)

    def parts(self):
        return [self.block] + list(self.named.values())

    def cache_parts(self):
        """(name, part) of the parts that keep a cache, in the plan's order."""
        return [(n, p) for n, p in self.named.items() if hasattr(p, "cache_need")]


class Model:
    def __init__(self, plan, config=None):
        plan.check()
        self.plan = plan
        self.config = config
        self.embedding = make_part("embedding", plan.embedding)
        self.layers = [Layer(lp.label, make_part("block", lp.block),
                             {name: make_part(role, spec) for name, role, spec in lp.parts}) for lp in plan.layers]
        self.final_norm = make_part("norm", plan.final_norm)
        self.head = make_part("head", plan.head)
        self.schedule = plan.schedule
        self.hidden_size = plan.hidden_size
        self.vocab_size = plan.vocab_size
        self.dtype = None
        self.device = None

    # ---- construction --------------------------------------------------
    @classmethod
    def from_config(cls, config):
        """Parts without tensors (enough to list them or to plan a cache)."""
        _, plan_fn = architecture(config.architecture)
        return cls(plan_fn(config), config)

    @classmethod
    def from_dir(cls, model_dir, dtype, ops, options=None):
        """``options``: model options of the session (``config.apply_model_options``)."""
        model = cls.from_config(read_config(model_dir, options))
        dt = compute_dtype(dtype)
        model._bind(load_tensors(model_dir, model.param_specs(), dt, ops.device), dt, ops)
        return model

    @classmethod
    def from_random(cls, config, seed, dtype, ops):
        """Random weights made on the device, without a file."""
        if isinstance(config, dict):
            config = config_from_dict(config)
        model = cls.from_config(config)
        dt = compute_dtype(dtype)
        model._bind(random_device_tensors(model.param_specs(), seed, dt, ops.device), dt, ops)
        return model

    def _all_parts(self):
        parts = [self.embedding]
        for layer in self.layers:
            parts.extend(layer.parts())
        return parts + [self.final_norm, self.head]

    @property
    def short_request_rows(self):
        """Requests that bring fewer tokens than this to a step are laid first in it (0: no such line): the largest
        that a part asks for (``Part.short_request_rows``)."""
        return max([getattr(p, "short_request_rows", 0) for p in self._all_parts()] + [0])

    def param_specs(self):
        specs, seen = [], set()
        for p in self._all_parts():
            for s in p.all_param_specs():
                if s.name in seen:
                    raise ValueError(f"two parts declare the tensor '{s.name}'")
                seen.add(s.name)
                specs.append(s)
        return specs

    def _bind(self, params, dtype, ops):
        self.dtype, self.device = dtype, ops.device
        for p in self._all_parts():
            p.bind_all(params, ops)

    @property
    def graph_safe(self):
        """Whether every part (and every part it owns) allows steps to be captured into graphs."""
        def safe(p):
            return p.graph_safe and all(safe(q) for q in p.sub_parts())
        return all(safe(p) for p in self._all_parts())

    # ---- what the cache manager needs to know -----------------------------
    def cache_needs(self):
        """One entry for every (schedule entry, part of its layer that keeps a cache): PagedKV,
        FixedState, or None (an entry that reads another entry's cache keeps none of its own).
        ``cache_slots[i]`` says which of them schedule entry ``i`` uses: {part name: index}."""
        needs, self.cache_slots = [], []
        for e in self.schedule:
            slots = {}
            for name, part in self.layers[e.layer].cache_parts():
                need = part.cache_need() if e.cache_of is None else None
                if need is not None and not isinstance(need, (PagedKV, FixedState)):
                    raise TypeError(f"{type(part).__name__}.cache_need() returned {need!r}")
                slots[name] = len(needs)
                needs.append(need)
            self.cache_slots.append(slots)
        return needs

    # ---- the forward pass of one step ----------------------------------------
    def forward(self, ops, step, caches, logits_out):
        """Runs ``step``'s tokens through the schedule. ``caches[k]`` is the cache view
        of entry ``k`` of ``cache_needs()`` (None if it needs none). Writes fp32 logits for
        ``step.logit_rows`` into ``logits_out`` ([R, V]; R may be 0)."""
        with ops.on_current_stream(), ops.section("total"):
            self._forward(ops, step, caches, logits_out)

    def _forward(self, ops, step, caches, logits_out):
        T = step.n_tokens
        x = ops.scratch("residual", (T, self.hidden_size), torch.float32)
        self.embedding.forward(ops, step, x)
        if not hasattr(self, "cache_slots"):
            self.cache_needs()
        for i, e in enumerate(self.schedule):
            layer = self.layers[e.layer]
            own = e.cache_of is None
            mine = {name: caches[k] for name, k in self.cache_slots[i if own else e.cache_of].items()}
            layer.block.forward(ops, step, x, layer.named, mine, write_cache=own)
        R = step.n_logit_rows
        if R:
            h = ops.scratch("head_in", (R, self.hidden_size), ops.act_dtype)
            if getattr(step, "rows_in_order", False):         # every token's logits, in order: no rows to gather
                norm_for(ops, self.final_norm, self.head, x, h)
            else:
                self.final_norm.forward(ops, x, h, rows=step.logit_rows)      # src/model.c:629-636
            self.head.forward(ops, h, logits_out)
        ops.settle()

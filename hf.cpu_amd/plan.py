"""A model described as data.

An architecture turns its typed configuration into a ``ModelPlan``: which parts
make up each layer (chosen layer by layer), what tensors they are called in the
checkpoint, and in which order the layers run. Everything downstream (the
loader, the random-weights writer, the cache manager, the step function) works
from the plan alone and never asks which architecture it came from.
"""
from dataclasses import dataclass, field
from typing import Optional


@dataclass(frozen=True)
class PartSpec:
    """One part: the registered ``kind`` under its role, and its sizes and
    constants, among them the ``prefix`` of its tensors' names if it has tensors.
    ``args`` may hold nested PartSpecs (a mixer's position encoding)."""
    kind: str
    args: dict = field(default_factory=dict)


@dataclass(frozen=True)
class LayerPlan:
    """One layer: ``block`` names the arrangement (where norms and residual sums sit, which
    branches there are) and ``parts`` the parts it arranges, as a mapping from the name the block
    knows a part by to ``(role, PartSpec)``. A block may have any number of parts of any role: four
    norms, two mixers side by side, no feed-forward. ``label`` is for messages only.

    ``LayerPlan.of(label, block, norm1=..., mixer=..., norm2=..., feed_forward=...)`` is the short
    way for the usual four: the role of a part is taken from its name (``norm*`` are norms)."""
    label: str
    block: PartSpec
    parts: tuple = ()            # of (name, role, PartSpec); a tuple so that the plan stays hashable

    @classmethod
    def of(cls, label, block, **named):
        """Parts by keyword; the role follows from the name: ``mixer*``, ``feed_forward*``, ``norm*``,
        ``position*``, or give ``name=(role, spec)``."""
        parts = []
        for name, spec in named.items():
            if isinstance(spec, tuple):
                role, spec = spec
            else:
                role = next((r for r in ("mixer", "feed_forward", "norm", "position") if name.startswith(r)), None)
                if role is None:
                    raise ValueError(f"layer {label!r}: the role of part '{name}' does not follow from its name; "
                                     f"give {name}=(role, spec)")
            parts.append((name, role, spec))
        return cls(label, block, tuple(parts))

    def part(self, name):
        for n, _, spec in self.parts:
            if n == name:
                return spec
        raise KeyError(f"layer {self.label!r} has no part '{name}'")

    def __getattr__(self, name):             # plan.layers[1].mixer, for the parts a layer has
        if name.startswith("_") or name in ("label", "block", "parts"):
            raise AttributeError(name)
        try:
            return self.part(name)
        except KeyError as e:
            raise AttributeError(str(e)) from None


@dataclass(frozen=True)
class ScheduleEntry:
    """One execution of a layer. Entries run in list order; a layer may appear more
    than once (each appearance has a cache of its own), and an entry with
    ``cache_of`` set keeps no cache but reads the one of that earlier entry."""
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelPlan:
    hidden_size: int
    vocab_size: int
    embedding: PartSpec          # role "embedding"
    layers: tuple                # of LayerPlan
    schedule: tuple              # of ScheduleEntry
    final_norm: PartSpec
    head: PartSpec               # role "head"
    max_context: int = 0         # trained context, informational (src/model.c:128-129)
    eos_token_ids: tuple = ()

    def check(self):
        n = len(self.layers)
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < n:
                raise ValueError(f"schedule entry {i} names layer {e.layer}, the plan has {n}")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_of}, "
                                     "which does not run before it")
                if self.schedule[e.cache_of].cache_of is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_of}, "
                                     "which keeps none of its own")
        return self

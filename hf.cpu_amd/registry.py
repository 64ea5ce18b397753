"""The registries: architecture name -> (configuration class, plan function), and
(role, kind) -> part class.

The architecture name is the string in config.json's ``architectures``; an
unknown one is refused by name, as the reference refuses an unknown
``general.architecture`` (src/model.c:107-110).
"""
from .status import ENOTSUP, fail

ROLES = ("embedding", "norm", "position", "mixer", "feed_forward", "block", "head")

_architectures = {}
_parts = {role: {} for role in ROLES}


def register_architecture(name, config_cls, plan_fn):
    """``config_cls.from_dict(obj, origin)`` reads config.json; ``plan_fn(config)``
    returns the ModelPlan. Registering a name again replaces the entry."""
    _architectures[name] = (config_cls, plan_fn)


def architecture(name):
    if name not in _architectures:
        known = ", ".join(sorted(_architectures)) or "none"
        fail(ENOTSUP, f"architecture '{name}' is not supported (registered: {known})")
    return _architectures[name]


def architectures():
    return sorted(_architectures)


def register_part(role, kind):
    """Class decorator: ``@register_part("mixer", "attention")``."""
    if role not in _parts:
        raise ValueError(f"unknown role '{role}' (roles: {', '.join(ROLES)})")

    def deco(cls):
        _parts[role][kind] = cls
        cls.role = role
        cls.kind = kind
        return cls
    return deco


def part_class(role, kind):
    if kind not in _parts[role]:
        known = ", ".join(sorted(_parts[role])) or "none"
        fail(ENOTSUP, f"no {role} part of kind '{kind}' is registered (registered: {known})")
    return _parts[role][kind]


def make_part(role, spec):
    """Builds the part that ``spec`` names from its arguments."""
    return part_class(role, spec.kind)(**spec.args)

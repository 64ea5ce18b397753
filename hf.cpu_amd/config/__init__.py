"""Reading a model folder's config.json into the typed configuration of its architecture."""
from ..registry import architecture
from ..status import EFORMAT, ENOTSUP, fail
from .reader import KeyReader, config_path, read_json_file
from .qwen2 import Qwen2Config


def config_from_dict(obj, origin="config.json"):
    """The typed configuration for ``obj['architectures'][0]``, by the registry."""
    names = KeyReader(obj, origin).str_list("architectures")
    if not names:
        fail(EFORMAT, f"{origin}: key 'architectures' is empty")
    config_cls, _ = architecture(names[0])
    return config_cls.from_dict(obj, origin)


def apply_model_options(obj, options, origin="config.json"):
    """``obj`` (a config.json object) with the session's model options applied. An option is a name and a
    value that the command line or a caller gives without knowing the architecture (``window``: the attention
    window in tokens, 0 for none); which keys of config.json it stands for is the business of the
    architecture's configuration class: ``config_cls.apply_options(obj, options)`` returns the changed
    object. An architecture without that method, or one that does not know an option, refuses it by name."""
    options = {k: v for k, v in (options or {}).items() if v is not None}
    if not options:
        return obj
    names = KeyReader(obj, origin).str_list("architectures")
    if not names:
        fail(EFORMAT, f"{origin}: key 'architectures' is empty")
    config_cls, _ = architecture(names[0])
    hook = getattr(config_cls, "apply_options", None)
    if hook is None:
        fail(ENOTSUP, f"architecture '{names[0]}' takes no model options (given: {', '.join(sorted(options))})")
    return hook(obj, options)


def read_config(model_dir, options=None):
    """The typed configuration of the folder's config.json; ``options`` (see ``apply_model_options``)
    change the file's keys before they are read and checked (the command line's ``--window``)."""
    path = config_path(model_dir)
    return config_from_dict(apply_model_options(read_json_file(path), options, path), path)


__all__ = ["KeyReader", "Qwen2Config", "apply_model_options", "config_from_dict", "read_config", "read_json_file"]

"""Reading a model folder's config.json into the typed configuration of its architecture."""
from ..registry import architecture
from ..status import EFORMAT, fail
from .reader import KeyReader, config_path, read_json_file
from .qwen2 import Qwen2Config


def config_from_dict(obj, origin="config.json"):
    """The typed configuration for ``obj['architectures'][0]``, by the registry."""
    names = KeyReader(obj, origin).str_list("architectures")
    if not names:
        fail(EFORMAT, f"{origin}: key 'architectures' is empty")
    config_cls, _ = architecture(names[0])
    return config_cls.from_dict(obj, origin)


def read_config(model_dir, overrides=None):
    """The typed configuration of the folder's config.json; ``overrides`` replaces keys of the file
    before they are read and checked (the command line's ``--window``)."""
    path = config_path(model_dir)
    obj = read_json_file(path)
    if overrides:
        obj = dict(obj, **overrides)
    return config_from_dict(obj, path)


__all__ = ["KeyReader", "Qwen2Config", "config_from_dict", "read_config", "read_json_file"]

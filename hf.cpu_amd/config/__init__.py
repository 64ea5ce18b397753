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


def read_config(model_dir):
    path = config_path(model_dir)
    return config_from_dict(read_json_file(path), path)


__all__ = ["KeyReader", "Qwen2Config", "config_from_dict", "read_config", "read_json_file"]

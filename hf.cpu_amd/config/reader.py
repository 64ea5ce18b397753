"""Typed access to the keys of a config.json.

The discipline is the reference's for GGUF metadata: a required key that is
missing is a format error naming the key (src/model.c:40-48), a value outside
its plausible range is a format error naming key and value (src/model.c:119-121),
an optional key falls back to its default without a message (src/model.c:126-139).
"""
import json
import os

from ..status import EFORMAT, EIO, fail

_MISSING = object()


class KeyReader:
    """Reads typed values out of one JSON object and remembers where it came from."""

    def __init__(self, obj, origin="config.json"):
        if not isinstance(obj, dict):
            fail(EFORMAT, f"{origin}: top level is not a JSON object")
        self.obj = obj
        self.origin = origin

    def has(self, key):
        return key in self.obj and self.obj[key] is not None

    def _get(self, key, default):
        if self.has(key):
            return self.obj[key]
        if default is _MISSING:
            fail(EFORMAT, f"{self.origin}: key '{key}' is missing")
        return default

    def integer(self, key, default=_MISSING, lo=1, hi=10 ** 6):
        v = self._get(key, default)
        if v is default and default is not _MISSING:
            return v
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v == int(v):
                v = int(v)
            else:
                fail(EFORMAT, f"{self.origin}: key '{key}' is not an integer: {v!r}")
        if not lo <= v <= hi:
            fail(EFORMAT, f"{self.origin}: key '{key}' has an implausible value {v} (allowed {lo}..{hi})")
        return v

    def number(self, key, default=_MISSING, lo=None, hi=None):
        v = self._get(key, default)
        if v is default and default is not _MISSING:
            return v
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            fail(EFORMAT, f"{self.origin}: key '{key}' is not a number: {v!r}")
        v = float(v)
        if v != v or (lo is not None and not v > lo) or (hi is not None and not v < hi):
            fail(EFORMAT, f"{self.origin}: key '{key}' has an implausible value {v}")
        return v

    def boolean(self, key, default=_MISSING):
        v = self._get(key, default)
        if not isinstance(v, bool):
            fail(EFORMAT, f"{self.origin}: key '{key}' is not true or false: {v!r}")
        return v

    def string(self, key, default=_MISSING):
        v = self._get(key, default)
        if v is default and default is not _MISSING:
            return v
        if not isinstance(v, str):
            fail(EFORMAT, f"{self.origin}: key '{key}' is not a string: {v!r}")
        return v

    def int_list(self, key, default=_MISSING):
        """A list of integers; a single integer counts as a list of one."""
        v = self._get(key, default)
        if v is default and default is not _MISSING:
            return v
        if isinstance(v, int) and not isinstance(v, bool):
            v = [v]
        if not isinstance(v, list) or any(isinstance(i, bool) or not isinstance(i, int) for i in v):
            fail(EFORMAT, f"{self.origin}: key '{key}' is not a list of integers: {v!r}")
        return tuple(v)

    def str_list(self, key, default=_MISSING):
        v = self._get(key, default)
        if v is default and default is not _MISSING:
            return v
        if not isinstance(v, list) or any(not isinstance(i, str) for i in v):
            fail(EFORMAT, f"{self.origin}: key '{key}' is not a list of strings: {v!r}")
        return tuple(v)


def read_json_file(path):
    """The parsed JSON of ``path``; EIO if it cannot be read, EFORMAT (with line and
    column) if it is not JSON."""
    try:
        with open(path, "rb") as f:
            raw = f.read()
    except OSError as e:
        fail(EIO, f"cannot read {path}: {e.strerror}")
    try:
        return json.loads(raw.decode("utf-8"))
    except UnicodeDecodeError as e:
        fail(EFORMAT, f"{path}: not UTF-8 at byte {e.start}")
    except json.JSONDecodeError as e:
        fail(EFORMAT, f"{path}: not JSON at line {e.lineno} column {e.colno} (byte {e.pos}): {e.msg}")


def config_path(model_dir):
    return os.path.join(model_dir, "config.json")

"""Import name for the package that lives in the folder ``hf.cpu_amd/``.

A folder name with a dot cannot be imported directly, so this module loads that
folder as the package ``hf_cpu_amd`` (sub-packages resolve inside the folder).
"""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hf.cpu_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_mod = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _mod
_spec.loader.exec_module(_mod)

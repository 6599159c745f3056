"""Loads the package directory `spirula-studio_amd/` (its name is not a Python identifier) as the
module `spirula_studio_amd`."""
import importlib.util
import os
import sys

_NAME = "spirula_studio_amd"


def load():
    if _NAME in sys.modules:
        return sys.modules[_NAME]
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "spirula-studio_amd")
    spec = importlib.util.spec_from_file_location(
        _NAME, os.path.join(root, "__init__.py"), submodule_search_locations=[root])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[_NAME] = mod
    spec.loader.exec_module(mod)
    return mod

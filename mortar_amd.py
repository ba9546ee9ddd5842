"""Import shim: exposes the package directory (whose name is not a Python identifier) as ``mortar_amd``."""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "morph-orchestrates-recursive-pruned-hierarchies_amd")
_spec = importlib.util.spec_from_file_location("mortar_amd", os.path.join(_dir, "__init__.py"),
                                               submodule_search_locations=[_dir])
_mod = importlib.util.module_from_spec(_spec)
sys.modules["mortar_amd"] = _mod
_spec.loader.exec_module(_mod)

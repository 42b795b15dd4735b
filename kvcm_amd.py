"""Import name of the package that lives in ``kv-cache-manager_amd/`` (a folder name Python
cannot import directly): ``import kvcm_amd`` loads that folder as the package ``kvcm_amd``."""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kv-cache-manager_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)

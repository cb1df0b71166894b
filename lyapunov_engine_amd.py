"""Import name of the package that lives in the folder ``lyapunov-engine_amd/``.

A folder name with a hyphen is not a Python identifier, so ``import
lyapunov_engine_amd`` lands here first; this module then loads the folder as
the package of that name and puts it in its own place in ``sys.modules``, so
that ``lyapunov_engine_amd.config`` and the other sub-packages resolve inside
the folder.
"""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lyapunov-engine_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir]
)
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)

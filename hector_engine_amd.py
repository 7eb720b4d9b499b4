"""Import shim: the package lives in the folder ``hector-engine_amd/`` whose
name is not a Python identifier.  ``import hector_engine_amd`` finds this file
and replaces itself in ``sys.modules`` with the package loaded from there, so
``hector_engine_amd.config`` and the other sub-packages import as usual."""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hector-engine_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)

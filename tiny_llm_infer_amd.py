"""Import shim: ``import tiny_llm_infer_amd`` loads the package that lives in
the folder ``tiny-llm-infer_amd/`` (a hyphen cannot appear in a Python module
name, so the folder is loaded under an importable name)."""
import importlib.util as _ilu
import os as _os
import sys as _sys

_pkg_dir = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "tiny-llm-infer_amd")
_spec = _ilu.spec_from_file_location(
    __name__, _os.path.join(_pkg_dir, "__init__.py"), submodule_search_locations=[_pkg_dir])
_module = _ilu.module_from_spec(_spec)
_sys.modules[__name__] = _module
_spec.loader.exec_module(_module)

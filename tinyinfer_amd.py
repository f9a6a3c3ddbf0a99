"""Import shim: `import tinyinfer_amd` loads the package that lives in the
folder `tinyinfer.cpp_amd/` (a folder name Python's import statement cannot
spell) and installs it in `sys.modules` under this name, sub-packages included.
"""
import importlib.util as _ilu
import os as _os
import sys as _sys

_here = _os.path.dirname(_os.path.abspath(__file__))
_pkg_dir = _os.path.join(_here, "tinyinfer.cpp_amd")
_spec = _ilu.spec_from_file_location(
    "tinyinfer_amd", _os.path.join(_pkg_dir, "__init__.py"),
    submodule_search_locations=[_pkg_dir])
_mod = _ilu.module_from_spec(_spec)
_sys.modules["tinyinfer_amd"] = _mod
_spec.loader.exec_module(_mod)

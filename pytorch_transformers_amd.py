"""Import name for the package whose folder is ``pytorch-transformers_amd``.

A hyphen is not allowed in a Python module name, so this file loads the
folder's ``__init__.py`` under the name ``pytorch_transformers_amd`` and puts
the result into ``sys.modules``; sub-packages (``.config``, ``.engine`` ...)
are then found in the folder as usual.
"""
import importlib.util as _ilu
import os as _os
import sys as _sys

_dir = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "pytorch-transformers_amd")
_spec = _ilu.spec_from_file_location(
    __name__, _os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir]
)
_mod = _ilu.module_from_spec(_spec)
_sys.modules[__name__] = _mod
_spec.loader.exec_module(_mod)

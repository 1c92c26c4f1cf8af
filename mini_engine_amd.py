"""Import alias for the package whose sources live in the folder ``mini-engine_amd/``.

That folder name is not a Python identifier, so ``import mini_engine_amd`` goes through this
file: it loads ``mini-engine_amd/__init__.py`` as the package ``mini_engine_amd`` (with the
folder as its search path for submodules) and puts it in ``sys.modules`` in place of itself.
"""

import importlib.util as _ilu
import os as _os
import sys as _sys

_dir = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "mini-engine_amd")
_spec = _ilu.spec_from_file_location(
    "mini_engine_amd", _os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir]
)
_pkg = _ilu.module_from_spec(_spec)
_sys.modules["mini_engine_amd"] = _pkg
_spec.loader.exec_module(_pkg)

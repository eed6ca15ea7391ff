"""Import name of the package that lives in the folder ``xyntetik-runner_amd``.

The folder's name is not an identifier, so this module loads the folder's
``__init__.py`` as the package ``xyntetik_runner_amd`` and puts it in its own
place in ``sys.modules``; ``import xyntetik_runner_amd.engine`` and
``python -m xyntetik_runner_amd`` then work as for any package.
"""
import importlib.util as _ilu
import os as _os
import sys as _sys

_root = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "xyntetik-runner_amd")
_spec = _ilu.spec_from_file_location(
    "xyntetik_runner_amd", _os.path.join(_root, "__init__.py"),
    submodule_search_locations=[_root])
_pkg = _ilu.module_from_spec(_spec)
_sys.modules["xyntetik_runner_amd"] = _pkg
_spec.loader.exec_module(_pkg)

"""Import name of the package that lives in the folder ``burn-transformers_amd``.

A hyphen cannot be part of a Python module name, so this module loads the folder's
``__init__.py`` under the importable name ``burn_transformers_amd`` and puts the package in
its own place in ``sys.modules``; ``import burn_transformers_amd.engine`` and the like then
resolve inside that folder.
"""

import importlib.util
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
_FOLDER = os.path.join(_HERE, "burn-transformers_amd")
_spec = importlib.util.spec_from_file_location(
    "burn_transformers_amd", os.path.join(_FOLDER, "__init__.py"),
    submodule_search_locations=[_FOLDER])
_package = importlib.util.module_from_spec(_spec)
sys.modules["burn_transformers_amd"] = _package
_spec.loader.exec_module(_package)

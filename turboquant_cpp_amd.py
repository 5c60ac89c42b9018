"""Import name for the package kept in the folder ``turboquant.cpp_amd/``.

A folder name with a dot in it cannot be imported by name, so this module
loads the folder's ``__init__.py`` under the name ``turboquant_cpp_amd`` and
replaces itself with the package.  ``import turboquant_cpp_amd.engine`` and
friends then resolve inside the folder.
"""
import importlib.util
import os
import sys

_PKG_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "turboquant.cpp_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_PKG_DIR, "__init__.py"), submodule_search_locations=[_PKG_DIR]
)
_pkg = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _pkg
_spec.loader.exec_module(_pkg)

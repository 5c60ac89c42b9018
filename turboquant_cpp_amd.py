"""Import name for the package kept in the folder ``turboquant.cpp_amd/``.

A folder name with a dot in it cannot be imported by name, so this module loads the folder's
``__init__.py`` under the name ``turboquant_cpp_amd`` and replaces itself with the package.
``import turboquant_cpp_amd.engine`` and friends then resolve inside the folder, and
``python -m turboquant_cpp_amd ...`` runs the command line (``cli.py``).
"""
import importlib.util
import os
import sys

_NAME = "turboquant_cpp_amd"
_PKG_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "turboquant.cpp_amd")


def _load_package():
    spec = importlib.util.spec_from_file_location(
        _NAME, os.path.join(_PKG_DIR, "__init__.py"), submodule_search_locations=[_PKG_DIR])
    pkg = importlib.util.module_from_spec(spec)
    sys.modules[_NAME] = pkg
    spec.loader.exec_module(pkg)
    return pkg


if __name__ == "__main__":
    _load_package()
    from turboquant_cpp_amd.cli import main
    sys.exit(main())
else:
    _load_package()

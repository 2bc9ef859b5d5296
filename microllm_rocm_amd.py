"""Import name for the package whose folder is ``microllm-rocm_amd/``.

The folder's name holds a hyphen, which Python cannot import, so this module
loads the folder's ``__init__.py`` under the name ``microllm_rocm_amd`` and puts
the package in its own place in ``sys.modules``.
"""
import importlib.util
import os
import sys

_folder = os.path.join(os.path.dirname(os.path.abspath(__file__)), "microllm-rocm_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_folder, "__init__.py"), submodule_search_locations=[_folder])
_package = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _package
_spec.loader.exec_module(_package)

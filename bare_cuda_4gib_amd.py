"""Import name of the framework.

The package folder is called ``bare-cuda-4gib_amd``, which is no Python
identifier; this module loads that folder as the package
``bare_cuda_4gib_amd`` so that ``import bare_cuda_4gib_amd.engine`` works.
"""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bare-cuda-4gib_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)

"""Import name of the package that lives in the folder `xeno-rt_amd/`.

A hyphen cannot appear in a Python module name, so `import xeno_rt_amd`
finds this file, and this file loads the folder as the package of that name.
"""
import importlib.util
import os
import sys

_folder = os.path.join(os.path.dirname(os.path.abspath(__file__)), "xeno-rt_amd")
_spec = importlib.util.spec_from_file_location(
    "xeno_rt_amd", os.path.join(_folder, "__init__.py"), submodule_search_locations=[_folder])
_package = importlib.util.module_from_spec(_spec)
sys.modules["xeno_rt_amd"] = _package
_spec.loader.exec_module(_package)

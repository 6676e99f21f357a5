"""Import name of the package. The package lives in the folder
`ninfer-amd-mi50_amd/`, whose name is not a Python identifier; this module
loads it under the name `ninfer_amd` and puts it in its own place."""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ninfer-amd-mi50_amd")
_spec = importlib.util.spec_from_file_location(
    "ninfer_amd", os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_module = importlib.util.module_from_spec(_spec)
sys.modules["ninfer_amd"] = _module
_spec.loader.exec_module(_module)

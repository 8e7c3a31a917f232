"""Import name of the package whose folder is `herbert-rs_amd/`.

A folder with a hyphen cannot be imported by name, so this module loads
`herbert-rs_amd/__init__.py` as the package `herbert_rs_amd` and puts it in
its own place in `sys.modules`; sub-modules are then found in that folder.
"""
import importlib.util
import os
import sys

_folder = os.path.join(os.path.dirname(os.path.abspath(__file__)), "herbert-rs_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_folder, "__init__.py"), submodule_search_locations=[_folder])
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)

"""Import name for the package that lives in the folder ``vipera.rs_amd/``.

A folder name with a dot cannot be written in an ``import`` statement, so this
module loads that folder as the package ``vipera_rs_amd`` and takes its place in
``sys.modules``.  After ``import vipera_rs_amd`` every submodule is reachable as
``vipera_rs_amd.<name>``.
"""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vipera.rs_amd")
_spec = importlib.util.spec_from_file_location(
    "vipera_rs_amd", os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir]
)
_module = importlib.util.module_from_spec(_spec)
sys.modules["vipera_rs_amd"] = _module
_spec.loader.exec_module(_module)

"""Makes the package directory ``llm-infer_amd`` importable as ``llm_infer_amd``.

A hyphen cannot stand in a module name, so this file loads the directory's
``__init__.py`` under the importable name and takes its place in ``sys.modules``.
"""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "llm-infer_amd")
_spec = importlib.util.spec_from_file_location(
    "llm_infer_amd", os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_module = importlib.util.module_from_spec(_spec)
sys.modules["llm_infer_amd"] = _module
_spec.loader.exec_module(_module)

"""Import alias: ``import gpt_neox_amd`` loads the package in ``gpt-neox_amd/``.

The package directory carries the project's name, which is not a valid Python
identifier; this module loads it from its path and installs it in ``sys.modules``
under ``gpt_neox_amd`` (replacing itself), so ``gpt_neox_amd.fused_softmax`` etc.
import normally afterwards.
"""
import importlib.util
import os
import sys

_pkg_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpt-neox_amd")
_spec = importlib.util.spec_from_file_location(
    "gpt_neox_amd", os.path.join(_pkg_dir, "__init__.py"), submodule_search_locations=[_pkg_dir]
)
_module = importlib.util.module_from_spec(_spec)
sys.modules["gpt_neox_amd"] = _module
_spec.loader.exec_module(_module)

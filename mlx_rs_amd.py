"""Import shim: the package directory is named ``mlx-rs_amd`` (not a Python identifier).

``import mlx_rs_amd`` executes this file, which loads ``mlx-rs_amd/__init__.py`` as the
package ``mlx_rs_amd`` and puts it in ``sys.modules`` in place of the shim.
"""
import importlib.util
import os
import sys

_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mlx-rs_amd")
_spec = importlib.util.spec_from_file_location(
    "mlx_rs_amd", os.path.join(_dir, "__init__.py"), submodule_search_locations=[_dir])
_mod = importlib.util.module_from_spec(_spec)
sys.modules["mlx_rs_amd"] = _mod
_spec.loader.exec_module(_mod)

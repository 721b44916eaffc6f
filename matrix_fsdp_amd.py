"""Import alias for the package directory ``matrix-fsdp_amd/``.

The directory name carries a hyphen and so is not a Python identifier; this
module loads it under the importable name ``matrix_fsdp_amd`` and replaces
itself in ``sys.modules`` with the real package, so that
``import matrix_fsdp_amd.kernels.native`` works with the repository root on
``sys.path``.
"""
import importlib.util
import os
import sys

_PKG_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "matrix-fsdp_amd")
_spec = importlib.util.spec_from_file_location(
    "matrix_fsdp_amd",
    os.path.join(_PKG_DIR, "__init__.py"),
    submodule_search_locations=[_PKG_DIR],
)
_module = importlib.util.module_from_spec(_spec)
sys.modules["matrix_fsdp_amd"] = _module
_spec.loader.exec_module(_module)

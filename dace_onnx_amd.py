"""Import alias: ``import dace_onnx_amd`` loads the package kept in ``dace-onnx_amd/``.

The directory name carries a hyphen (it is named after the project), which is
not a valid Python identifier; this module replaces itself in ``sys.modules``
with the package found there so that ``dace_onnx_amd.onnx`` etc. resolve
normally.
"""
import importlib.util
import os
import sys

_pkg_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dace-onnx_amd")
_spec = importlib.util.spec_from_file_location(
    __name__, os.path.join(_pkg_dir, "__init__.py"), submodule_search_locations=[_pkg_dir])
_module = importlib.util.module_from_spec(_spec)
sys.modules[__name__] = _module
_spec.loader.exec_module(_module)

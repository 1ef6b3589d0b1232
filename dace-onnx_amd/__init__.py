"""MI355X-native expansions for DaCeML's ONNX library nodes.

Layout (mirrors the part of ``daceml`` that lies on the expansion hot path):

``csrc/``                       HIP kernels (gfx950) and the C ABI, built into ``libmi355x_onnx.so``
``_lib``                        ctypes binding of that library
``sdfg``                        the small slice of the DaCe graph API the expansions are written against
``onnx``                        ``ONNXForward`` registry, ``ONNX<Op>`` library nodes, the ``"mi355x"``
                                implementations and the ``ONNXModel`` runner (``import dace_onnx_amd.onnx as donnx``)
``util``                        ``in_desc_with_name`` / ``expand_onnx_nodes`` / ``auto_optimize``
``testing``                     ``torch_tensors_close``; ``testing.profiling``: HIP-event timers
"""
import logging
import os

log = logging.getLogger(__name__)
log.setLevel(os.environ.get("DACEML_LOG_LEVEL", "WARNING"))  # same switch as daceml/__init__.py:9-11

from . import _lib  # noqa: E402,F401
from . import sdfg  # noqa: E402,F401

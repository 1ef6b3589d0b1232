"""``import dace_onnx_amd.onnx as donnx`` -- the counterpart of ``daceml.onnx``.

``donnx.ONNX<Op>`` are the library nodes, ``donnx.default_implementation`` is the
library-wide default (the reference sets ``"onnxruntime"`` in
``daceml/onnx/__init__.py:8``; here it is ``"mi355x"``), ``donnx.ONNXModel`` runs
an ONNX graph.
"""
from .schema import ONNXAttributeType, ONNXAttribute, ONNXTypeConstraint, ONNXParameterType, ONNXSchema, \
    ONNXParameter
from .nodes import *  # noqa: F401,F403
from .nodes import ONNXOp, has_onnx_node, get_onnx_node, ExpansionRefused
from .forward_implementation_abc import ONNXForward
from . import op_implementations
from .op_implementations.utils import op_implementation

#: implementation used when neither the node nor its class names one
default_implementation = "mi355x"

from .onnx_importer import ONNXModel  # noqa: E402

from .onnx_op import *  # noqa: F401,F403
from .onnx_op import ONNXOp, has_onnx_node, get_onnx_node, bind_implementation, ExpansionRefused, \
    ExpandTransformation, expand_node

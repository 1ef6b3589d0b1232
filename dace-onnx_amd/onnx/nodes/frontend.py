"""Call form of the ONNX nodes: ``donnx.ONNXMatMul(A=a, B=b, Y=y)``.

In the reference this spelling is only legal inside a ``@dace.program``, where
the DaCe Python frontend rewrites it into a library node with one access node
per keyword (``daceml/onnx/nodes/onnx_op.py:420-475``). Here the same keyword
split (attributes / inputs / outputs by schema, ``TypeError`` on anything else)
builds a one-node SDFG, expands it and runs it immediately on the GPU; outputs
are written into the tensors or arrays the caller passed.
"""
import numpy as np

from ... import sdfg as dace
from .node_utils import parse_variadic_param


def call_onnx_op(cls, **kwargs):
    schema = cls.schema
    attrs = {k: v for k, v in kwargs.items() if k in schema.attributes}
    kwargs = {k: v for k, v in kwargs.items() if k not in attrs}

    def pick(names, variadic):
        return {k: v for k, v in kwargs.items()
                if k in names or ("__" in k and parse_variadic_param(k)[0] in variadic)}

    inputs = pick(schema.non_variadic_inputs(), schema.variadic_inputs())
    kwargs = {k: v for k, v in kwargs.items() if k not in inputs}
    outputs = pick(schema.non_variadic_outputs(), schema.variadic_outputs())
    kwargs = {k: v for k, v in kwargs.items() if k not in outputs}
    if len(kwargs) > 0:
        raise TypeError(f"Unknown arguments {', '.join(kwargs)}")

    sdfg = dace.SDFG("call_" + schema.name)
    state = sdfg.add_state()
    node = object.__new__(cls)
    cls.__init__(node, "ONNX" + schema.name, **attrs)
    state.add_node(node)
    call_args = {}
    # small host integer arrays (Slice's starts / ends / axes / steps, a Reshape target) are compile-time
    # constants of this one-node graph, as initializers are in an imported model
    sdfg._constant_inputs = {}
    for conn, value in list(inputs.items()) + list(outputs.items()):
        arr = "__" + conn
        if conn in inputs and isinstance(value, np.ndarray) and np.issubdtype(value.dtype, np.integer) and value.size <= 64:
            sdfg._constant_inputs[arr] = value.copy()
        shape = tuple(value.shape) if hasattr(value, "shape") else ()
        dtype = value.dtype if hasattr(value, "dtype") else np.asarray(value).dtype
        sdfg.add_array(arr, shape, dace.typeclass_of(dtype))
        call_args[arr] = value
        if conn in inputs:
            state.add_edge(state.add_read(arr), None, node, conn, sdfg.make_array_memlet(arr))
            node.add_in_connector(conn)
        else:
            state.add_edge(node, conn, state.add_write(arr), None, sdfg.make_array_memlet(arr))
            node.add_out_connector(conn)
    sdfg.expand_library_nodes()
    sdfg.compile()(**call_args)
    return None

"""Helpers for writing expansions (``daceml/onnx/op_implementations/utils.py``)."""
import copy

from ... import sdfg as dace
from ...sdfg import SDFG, SDFGState
from ..forward_implementation_abc import ONNXForward
from ...util.utils import in_desc_with_name, out_desc_with_name


def op_implementation(op, name):
    """A decorator that registers an op implementation.

    Use it on classes that extend :class:`ONNXForward`
    (same signature and docstring side effect as ``op_implementations/utils.py:17-38``).

    :param op: the ONNX name of the op to register for.
    :param name: the name of the implementation.
    """
    def dec(cls):
        note = """
                :Implementation name: ``"{}"``
                """.format(name)
        cls.__doc__ = (cls.__doc__ or "") + note
        ONNXForward.register(cls, op=op, name=name)
        return cls

    return dec


def empty_sdfg_for_node(sdfg: SDFG, state: SDFGState, node, add_access_nodes=True):
    """An SDFG usable as the nested-SDFG expansion of ``node``: one non-transient
    array per connected connector, named like the connector, with the descriptor
    taken from the node's edges (``op_implementations/utils.py:94-128``).

    :return: (nsdfg, nstate, input access nodes, output access nodes)
    """
    nsdfg = SDFG(node.label + "_expansion")
    nstate = nsdfg.add_state()
    input_nodes, output_nodes = {}, {}
    for edge, is_input in node.iter_edges(state):
        if is_input:
            conn_name = edge.dst_conn
            nsdfg.add_datadesc(conn_name, copy.deepcopy(in_desc_with_name(node, state, sdfg, conn_name)))
            if add_access_nodes:
                input_nodes[conn_name] = nstate.add_read(conn_name)
        else:
            conn_name = edge.src_conn
            nsdfg.add_datadesc(conn_name, copy.deepcopy(out_desc_with_name(node, state, sdfg, conn_name)))
            if add_access_nodes:
                output_nodes[conn_name] = nstate.add_write(conn_name)
        nsdfg.arrays[conn_name].transient = False
    return nsdfg, nstate, input_nodes, output_nodes


def kernel_call_for_node(node, state: SDFGState, function: str, args) -> dace.KernelCall:
    """A :class:`KernelCall` carrying exactly the connectors ``node`` has edges on."""
    inputs = [e.dst_conn for e in state.in_edges(node)]
    outputs = [e.src_conn for e in state.out_edges(node)]
    return dace.KernelCall(node.label + "_mi355x", function, args, inputs, outputs)

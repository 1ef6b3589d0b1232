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
    access = {True: {}, False: {}}   # is_input -> connector -> access node
    for edge, is_input in node.iter_edges(state):
        connector = edge.dst_conn if is_input else edge.src_conn
        outer = (in_desc_with_name if is_input else out_desc_with_name)(node, state, sdfg, connector)
        inner = copy.deepcopy(outer)
        inner.transient = False
        nsdfg.add_datadesc(connector, inner)
        if add_access_nodes:
            access[is_input][connector] = (nstate.add_read if is_input else nstate.add_write)(connector)
    return nsdfg, nstate, access[True], access[False]


def kernel_call_for_node(node, state: SDFGState, function: str, args) -> dace.KernelCall:
    """A :class:`KernelCall` carrying exactly the connectors ``node`` has edges on."""
    inputs = [e.dst_conn for e in state.in_edges(node)]
    outputs = [e.src_conn for e in state.out_edges(node)]
    return dace.KernelCall(node.label + "_mi355x", function, args, inputs, outputs)

"""Graph helpers used by expansions and by their caller
(``daceml/util/utils.py:34-55,156-222``)."""
import functools
import logging
import typing

from ..sdfg import SDFG, SDFGState, Node, MultiConnectorEdge, Array, NestedSDFG

log = logging.getLogger(__name__)


def in_edge_with_name(node: Node, state: SDFGState, name: str) -> MultiConnectorEdge:
    """Find the edge that connects to input connector ``name`` on ``node``."""
    cands = list(e for e in state.in_edges(node) if e.dst_conn == name)
    if len(cands) != 1:
        raise ValueError("Expected to find exactly one edge with name '{}', found {}".format(name, len(cands)))
    return cands[0]


def out_edge_with_name(node: Node, state: SDFGState, name: str) -> MultiConnectorEdge:
    """Find the edge that connects to output connector ``name`` on ``node``."""
    cands = list(e for e in state.out_edges(node) if e.src_conn == name)
    if len(cands) != 1:
        raise ValueError("Expected to find exactly one edge with name '{}', found {}".format(name, len(cands)))
    return cands[0]


def in_desc_with_name(node: Node, state: SDFGState, sdfg: SDFG, name: str) -> Array:
    """Descriptor of the data connected to input connector ``name``."""
    return sdfg.arrays[in_edge_with_name(node, state, name).data.data]


def out_desc_with_name(node: Node, state: SDFGState, sdfg: SDFG, name: str) -> Array:
    """Descriptor of the data connected to output connector ``name``."""
    return sdfg.arrays[out_edge_with_name(node, state, name).data.data]


def iterables_equal(a, b) -> bool:
    """Return whether the two iterables ``a`` and ``b`` are equal."""
    a, b = list(a), list(b)
    return len(a) == len(b) and all(x == y for x, y in zip(a, b))


def prod(sequence):
    return functools.reduce(lambda a, b: a * b, sequence, 1)


def is_cuda(storage) -> bool:
    """Check if a descriptor storage type is a GPU array."""
    return storage in ("GPU_Global", "GPU_Shared")


def expand_onnx_nodes(sdfg: SDFG, predicate: typing.Optional[typing.Callable[[Node], bool]] = None):
    """Expand all ONNX library nodes in ``sdfg``, nested SDFGs included
    (``daceml/util/utils.py:156-185``).

    :param predicate: only nodes for which ``predicate(node)`` is true are expanded.
    """
    from ..onnx.nodes.onnx_op import ONNXOp
    if predicate is None:
        def predicate(n):
            return True
    expanded_something = True
    while expanded_something:
        expanded_something = False
        for st in sdfg.nodes():
            for node in st.nodes():
                if isinstance(node, NestedSDFG):
                    expand_onnx_nodes(node.sdfg, predicate=predicate)
                elif isinstance(node, ONNXOp) and predicate(node):
                    impl_name = node.expand(sdfg, st)
                    log.info("Expanded library node '%s' with implementation '%s'", node.label, impl_name)
                    expanded_something = True


def auto_optimize(sdfg: SDFG, cuda: bool = True, apply_strict: bool = False, fuse: bool = True):
    """Prepare an ONNX SDFG for execution (``daceml/util/utils.py:188-222``).

    The reference expands the ONNX nodes and then switches DaCe's BLAS nodes to
    their fast library implementations. Here there is one fast implementation
    per node, so the step that matters is graph-level fusion before expansion:
    bias / activation / residual nodes are folded into the contraction that
    feeds them and Reshape+Transpose pairs around attention become strides
    (see ``dace_onnx_amd.transformation``).
    """
    if fuse:
        from ..transformation import fuse_onnx_graph
        fuse_onnx_graph(sdfg)
    expand_onnx_nodes(sdfg)

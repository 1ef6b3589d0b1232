"""Register the "mi355x" implementations with a real DaCeML installation.

Everything else in this package mirrors the reference's plugin interface so that it
runs without ``dace``; this module is the other direction: where ``dace`` and
``daceml`` are importable, ``register()`` adds ``"mi355x"`` to the reference's own
``ONNX<Op>`` library nodes, as out-of-tree code has to (the reference binds
implementations in a loop that has already run at import,
``daceml/onnx/nodes/onnx_op.py:646-687``; an external implementation repeats
``:652-683`` and calls ``register_implementation``).

How an expansion is produced: the DaCe node, its state and SDFG are *mirrored* into
this package's light objects (same connector names, attribute values, shapes,
strides, dtypes), the package's own expansion runs on the mirror and yields a
``KernelCall``; its ``as_cpp()`` text becomes the body of a C++ tasklet inside the
nested SDFG that ``empty_sdfg_for_node`` builds
(``daceml/onnx/op_implementations/utils.py:94-128``), exactly the shape of
``CudnnConvolution.forward`` (``cudnn_implementations.py:303-334``). The ``MI355X``
environment points DaCe's build at ``include/mi355x_onnx.h`` and
``libmi355x_onnx.so`` (modelled on ``daceml/onnx/environments/cudnn.py:11-67``).

``mirror_expansion`` depends only on attribute access (``state.in_edges``,
``edge.dst_conn``, ``edge.data.data``, ``sdfg.arrays``, ``desc.shape`` ...) and is
exercised by the test-suite on this package's own objects; ``register()`` needs the
real packages and raises ``ImportError`` naming what is missing otherwise.
"""
import os
import typing

from . import sdfg as light
from .onnx.forward_implementation_abc import ONNXForward as LightForward
from .onnx.nodes.onnx_op import get_onnx_node as light_node_class, has_onnx_node

IMPLEMENTATION_NAME = "mi355x"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _light_dtype(dtype):
    """This package's typeclass for a dace typeclass / numpy dtype (matched by name)."""
    name = getattr(dtype, "to_string", lambda: None)() or getattr(getattr(dtype, "type", None), "__name__", None) or str(dtype)
    return getattr(light, {"float": "float32", "double": "float64", "int": "int32"}.get(name, name))


def mirror_expansion(node, state, sdfg) -> typing.Optional[light.KernelCall]:
    """Run this package's "mi355x" expansion of ``node`` (an ``ONNX<Op>`` library node of
    DaCeML, or of this package) on a mirror of its surroundings. Returns the KernelCall, an
    ``AliasNode`` for view-only ops, or None when the implementation refuses the node."""
    op = node.schema.name
    if not has_onnx_node(op):
        return None
    impls = dict(LightForward.registered_implementations(op))
    if IMPLEMENTATION_NAME not in impls:
        return None
    attrs = {a: getattr(node, a) for a in node.schema.attributes if getattr(node, a, None) is not None}
    m_sdfg = light.SDFG(node.label + "_mirror")
    m_state = m_sdfg.add_state()
    m_node = light_node_class(op)(node.label, **attrs)
    m_state.add_node(m_node)
    for e in state.in_edges(node):
        if e.dst_conn is None:
            continue
        d = sdfg.arrays[e.data.data]
        m_sdfg.add_array(e.dst_conn, list(d.shape), _light_dtype(d.dtype), strides=list(d.strides), transient=False)
        m_node.add_in_connector(e.dst_conn)
        m_state.add_edge(m_state.add_access(e.dst_conn), None, m_node, e.dst_conn, m_sdfg.make_array_memlet(e.dst_conn))
    for e in state.out_edges(node):
        if e.src_conn is None:
            continue
        d = sdfg.arrays[e.data.data]
        m_sdfg.add_array(e.src_conn, list(d.shape), _light_dtype(d.dtype), strides=list(d.strides), transient=False)
        m_node.add_out_connector(e.src_conn)
        m_state.add_edge(m_node, e.src_conn, m_state.add_access(e.src_conn), None, m_sdfg.make_array_memlet(e.src_conn))
    impl = impls[IMPLEMENTATION_NAME]
    if not impl.forward_can_be_applied(m_node, m_state, m_sdfg):
        return None
    return impl.forward(m_node, m_state, m_sdfg)


def register(ops: typing.Optional[typing.Iterable[str]] = None) -> typing.List[str]:
    """Add ``"mi355x"`` to DaCeML's ``ONNX<Op>`` nodes. Returns the ops registered."""
    try:
        import dace
        import dace.library
        from dace.transformation.transformation import ExpandTransformation
    except ImportError as e:
        raise ImportError("daceml_adapter.register() needs the 'dace' package (the reference pins git 4c6a674)") from e
    try:
        import daceml.onnx as donnx
        from daceml.onnx.forward_implementation_abc import ONNXForward
        from daceml.onnx.op_implementations.utils import empty_sdfg_for_node
        from daceml.onnx.nodes.node_codegen import expand_node
    except ImportError as e:
        raise ImportError("daceml_adapter.register() needs the 'daceml' package (spcl/dace-onnx)") from e

    @dace.library.environment
    class MI355X:
        cmake_minimum_version = None
        cmake_packages = []
        cmake_variables = {}
        cmake_includes = [os.path.join(ROOT, "include")]
        cmake_libraries = [os.path.join(ROOT, "dace-onnx_amd", "libmi355x_onnx.so")]
        cmake_compile_flags = []
        cmake_link_flags = []
        cmake_files = []
        state_fields = []
        dependencies = []
        headers = ["mi355x_onnx.h"]
        init_code = ""
        finalize_code = ""

    def make_forward(op):
        class Impl(ONNXForward):
            environments = [MI355X]

            @staticmethod
            def forward_can_be_applied(node, state, sdfg):
                # the kernels take device pointers: every array the node touches has to live in GPU memory
                touched = [e.data.data for e in list(state.in_edges(node)) + list(state.out_edges(node))
                           if e.data is not None and e.data.data is not None]
                if any(sdfg.arrays[name].storage != dace.StorageType.GPU_Global for name in touched):
                    return False
                return isinstance(mirror_expansion(node, state, sdfg), light.KernelCall)

            @staticmethod
            def forward(node, state, sdfg):
                call = mirror_expansion(node, state, sdfg)
                nsdfg, nstate, inputs, outputs = empty_sdfg_for_node(sdfg, state, node)
                ptr = lambda conn: dace.pointer(nsdfg.arrays[conn].dtype)
                used_in = [c for c in inputs if any(isinstance(a, light.Ptr) and a.connector == c for a in call.args)]
                tasklet = nstate.add_tasklet(node.label + "_mi355x", {"_" + c: ptr(c) for c in used_in},
                                             {"_" + c: ptr(c) for c in outputs}, call.as_cpp(), dace.dtypes.Language.CPP)
                for c in used_in:
                    nstate.add_edge(inputs[c], None, tasklet, "_" + c, nsdfg.make_array_memlet(c))
                for c in outputs:
                    nstate.add_edge(tasklet, "_" + c, outputs[c], None, nsdfg.make_array_memlet(c))
                return nsdfg

        Impl.__name__ = Impl.__qualname__ = "MI355X" + op
        return Impl

    registered = []
    for op in (ops or ["MatMul", "Gemm", "Conv", "MatMulInteger", "Softmax", "Add", "Sub", "Mul", "Div", "Pow", "Relu", "Erf",
                       "Sqrt", "Log", "Tanh", "Sigmoid", "Softplus", "Reciprocal", "Exp", "Neg", "Abs", "ReduceMean", "ReduceSum",
                       "ReduceMax", "ReduceMin", "LogSoftmax", "Sum", "Cast", "Slice", "Einsum", "MaxPool", "GlobalAveragePool",
                       "BatchNormalization", "Squeeze", "Unsqueeze", "Transpose"]):
        dace_node = getattr(donnx, "ONNX" + op, None)
        if dace_node is None:
            continue
        impl = make_forward(op)

        # onnx_op.py:652-683, for one implementation
        class Expansion(ExpandTransformation):
            environments = list(getattr(impl, "environments", []))
            forward_impl = impl

            @classmethod
            def expansion(cls, node, state, sdfg):
                node.validate(sdfg, state)
                if cls.forward_impl.forward_can_be_applied(node, state, sdfg):
                    result = cls.forward_impl.forward(node, state, sdfg)
                    if hasattr(cls.forward_impl, "post_parse"):
                        cls.forward_impl.post_parse(node, state, sdfg, result)
                    return result
                return expand_node(node, state, sdfg)   # the reference's fallback: ONNX Runtime

        Expansion.__name__ = Expansion.__qualname__ = "Expansion_" + impl.__name__
        dace_node.register_implementation(IMPLEMENTATION_NAME, Expansion)
        registered.append(op)
    return registered

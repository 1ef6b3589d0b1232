"""``daceml_adapter.register()`` executed on the CPU against stand-ins for ``dace`` and ``daceml``.

Neither package can be installed here, so the code below the adapter's import guard would
otherwise never run. The stand-ins carry only what ``register()`` touches: the
``dace.library.environment`` decorator, ``ExpandTransformation``, ``StorageType``,
``dace.pointer``, ``dace.dtypes.Language``, two ``ONNX<Op>`` classes with
``register_implementation``, ``ONNXForward``, ``empty_sdfg_for_node`` and ``expand_node``.
The reference tests its own ORT bridge with monkey-patched fakes the same way
(``tests/test_input_outputs.py:25-38``). What is checked is the contract of
``daceml/onnx/nodes/onnx_op.py:646-687`` for an out-of-tree implementation.
"""
import os
import sys
import types

import pytest

import dace_onnx_amd.onnx as light_onnx
from dace_onnx_amd import _lib, daceml_adapter, sdfg as light
from dace_onnx_amd.onnx.op_implementations.utils import empty_sdfg_for_node as light_empty_sdfg_for_node


class _Tasklet(light.Node):
    def __init__(self, label, inputs, outputs, code, language):
        super().__init__(label, list(inputs), list(outputs))
        self.in_types, self.out_types = dict(inputs), dict(outputs)
        self.code, self.language = code, language


@pytest.fixture
def fake_daceml(monkeypatch):
    """Installs the stand-in modules and returns a namespace with what the assertions need."""
    ns = types.SimpleNamespace(fallbacks=[], environments=[])

    dace = types.ModuleType("dace")
    dace.StorageType = light.StorageType
    dace.pointer = lambda dtype: ("pointer", dtype)
    dace.dtypes = types.ModuleType("dace.dtypes")
    dace.dtypes.Language = types.SimpleNamespace(CPP="CPP", Python="Python")
    dace.library = types.ModuleType("dace.library")

    def environment(cls):
        cls._dace_library_environment = True
        ns.environments.append(cls)
        return cls

    dace.library.environment = environment
    dace.transformation = types.ModuleType("dace.transformation")
    dace.transformation.transformation = types.ModuleType("dace.transformation.transformation")

    class ExpandTransformation:
        environments = []

        @classmethod
        def expansion(cls, node, state, sdfg):
            raise NotImplementedError

    dace.transformation.transformation.ExpandTransformation = ExpandTransformation

    daceml = types.ModuleType("daceml")
    donnx = types.ModuleType("daceml.onnx")
    # node classes of their own (own implementation tables), same schema and validate() as the package's
    donnx.ONNXSoftmax = type("ONNXSoftmax", (light_onnx.ONNXSoftmax,), {})
    donnx.ONNXConv = type("ONNXConv", (light_onnx.ONNXConv,), {})
    abc_mod = types.ModuleType("daceml.onnx.forward_implementation_abc")

    class ONNXForward:
        @staticmethod
        def forward_can_be_applied(node, state, sdfg):
            return True

    abc_mod.ONNXForward = ONNXForward
    impls_mod = types.ModuleType("daceml.onnx.op_implementations")
    utils_mod = types.ModuleType("daceml.onnx.op_implementations.utils")

    def empty_sdfg_for_node(sdfg, state, node):
        nsdfg, nstate, inputs, outputs = light_empty_sdfg_for_node(sdfg, state, node)

        def add_tasklet(label, tin, tout, code, language):
            return nstate.add_node(_Tasklet(label, tin, tout, code, language))

        nstate.add_tasklet = add_tasklet
        return nsdfg, nstate, inputs, outputs

    utils_mod.empty_sdfg_for_node = empty_sdfg_for_node
    nodes_mod = types.ModuleType("daceml.onnx.nodes")
    codegen_mod = types.ModuleType("daceml.onnx.nodes.node_codegen")

    def expand_node(node, state, sdfg):
        ns.fallbacks.append(node.label)
        return "onnxruntime-expansion"

    codegen_mod.expand_node = expand_node

    modules = {"dace": dace, "dace.dtypes": dace.dtypes, "dace.library": dace.library,
               "dace.transformation": dace.transformation,
               "dace.transformation.transformation": dace.transformation.transformation,
               "daceml": daceml, "daceml.onnx": donnx, "daceml.onnx.forward_implementation_abc": abc_mod,
               "daceml.onnx.op_implementations": impls_mod, "daceml.onnx.op_implementations.utils": utils_mod,
               "daceml.onnx.nodes": nodes_mod, "daceml.onnx.nodes.node_codegen": codegen_mod}
    daceml.onnx = donnx
    donnx.forward_implementation_abc, donnx.op_implementations, donnx.nodes = abc_mod, impls_mod, nodes_mod
    impls_mod.utils, nodes_mod.node_codegen = utils_mod, codegen_mod
    for name, mod in modules.items():
        monkeypatch.setitem(sys.modules, name, mod)
    ns.dace, ns.donnx, ns.ExpandTransformation, ns.ONNXForward = dace, donnx, ExpandTransformation, ONNXForward
    return ns


def _wire(node, inputs, outputs, storage=light.StorageType.GPU_Global):
    sdfg = light.SDFG("outer")
    st = sdfg.add_state()
    st.add_node(node)
    for conn, shape in inputs.items():
        sdfg.add_array("in_" + conn, shape, light.float32, storage=storage)
        node.add_in_connector(conn)
        st.add_edge(st.add_read("in_" + conn), None, node, conn, sdfg.make_array_memlet("in_" + conn))
    for conn, shape in outputs.items():
        sdfg.add_array("out_" + conn, shape, light.float32, storage=storage)
        node.add_out_connector(conn)
        st.add_edge(node, conn, st.add_write("out_" + conn), None, sdfg.make_array_memlet("out_" + conn))
    return sdfg, st


def test_register_binds_expansions_to_the_daceml_node_classes(fake_daceml):
    ns = fake_daceml
    # ops DaCeML has no node class for are skipped; the rest are returned in the order asked for
    assert daceml_adapter.register(["Softmax", "NoSuchOp", "Conv"]) == ["Softmax", "Conv"]
    for cls in (ns.donnx.ONNXSoftmax, ns.donnx.ONNXConv):
        expansion = cls.implementations[daceml_adapter.IMPLEMENTATION_NAME]
        assert issubclass(expansion, ns.ExpandTransformation)
        assert issubclass(expansion.forward_impl, ns.ONNXForward)
        assert expansion.__name__ == "Expansion_MI355X" + cls.__name__[4:]
        # the expansion carries the implementation's environments (onnx_op.py:664-666)
        (env,) = expansion.environments
        assert env._dace_library_environment and env.headers == ["mi355x_onnx.h"]
        assert os.path.isfile(os.path.join(env.cmake_includes[0], "mi355x_onnx.h"))
        assert env.cmake_libraries == [_lib.LIBRARY_PATH]
    # the package's own node classes are untouched: their table still holds this package's expansion only
    assert light_onnx.ONNXSoftmax.implementations is not ns.donnx.ONNXSoftmax.implementations
    # one environment class per register() call, shared by every op
    assert len(ns.environments) == 1


def test_registered_expansion_builds_the_cpp_tasklet(fake_daceml):
    ns = fake_daceml
    daceml_adapter.register(["Softmax", "Conv"])
    node = ns.donnx.ONNXConv("conv", strides=[2, 2])
    sdfg, st = _wire(node, {"X": [5, 3, 10, 10], "W": [16, 3, 3, 3]}, {"Y": [5, 16, 4, 4]})
    expansion = ns.donnx.ONNXConv.implementations["mi355x"]
    nsdfg = expansion.expansion(node, st, sdfg)
    assert ns.fallbacks == []
    # arrays of the nested SDFG are named like the connectors and are not transient (utils.py:94-128)
    assert sorted(nsdfg.arrays) == ["W", "X", "Y"] and not any(d.transient for d in nsdfg.arrays.values())
    (nstate,) = nsdfg.nodes()
    (tasklet,) = [n for n in nstate.nodes() if isinstance(n, _Tasklet)]
    assert tasklet.label == "conv_mi355x" and tasklet.language == "CPP"
    # the body is the text the package's own expansion prints for the same node
    assert tasklet.code == daceml_adapter.mirror_expansion(node, st, sdfg).as_cpp()
    assert "mi355x_conv2d_f32(_X, _W, nullptr, _Y, 5, 3, 10, 10, 16, 3, 3" in tasklet.code
    assert "__dace_current_stream" in tasklet.code
    # connectors are pointer-typed and named _<connector> (cudnn_implementations.py:324-327)
    assert tasklet.in_types == {"_X": ("pointer", light.float32), "_W": ("pointer", light.float32)}
    assert tasklet.out_types == {"_Y": ("pointer", light.float32)}
    wired_in = sorted((e.src.data, e.dst_conn) for e in nstate.in_edges(tasklet))
    wired_out = sorted((e.src_conn, e.dst.data) for e in nstate.out_edges(tasklet))
    assert wired_in == [("W", "_W"), ("X", "_X")] and wired_out == [("_Y", "Y")]

    soft = ns.donnx.ONNXSoftmax("sm", axis=-1)
    sdfg, st = _wire(soft, {"input": [4, 128]}, {"output": [4, 128]})
    nsdfg = ns.donnx.ONNXSoftmax.implementations["mi355x"].expansion(soft, st, sdfg)
    (tasklet,) = [n for n in nsdfg.nodes()[0].nodes() if isinstance(n, _Tasklet)]
    assert "mi355x_softmax_f32(_input, _output, 4, 128, 1, __dace_current_stream)" in tasklet.code


def test_registered_expansion_wires_only_the_inputs_the_call_reads(fake_daceml, monkeypatch):
    ns = fake_daceml
    daceml_adapter.register(["Conv"])
    node = ns.donnx.ONNXConv("conv")
    sdfg, st = _wire(node, {"X": [1, 32, 8, 8], "W": [32, 32, 1, 1], "B": [32]}, {"Y": [1, 32, 8, 8]})
    real = daceml_adapter.mirror_expansion(node, st, sdfg)
    assert any(isinstance(a, light.Ptr) and a.connector == "B" for a in real.args)
    # an expansion that consumes an input at expansion time (no pointer to it in the call) leaves it unconnected:
    # DaCe rejects a tasklet connector nothing reads
    without_b = light.KernelCall(real.label, real.function,
                                 [light.Ptr(None) if isinstance(a, light.Ptr) and a.connector == "B" else a
                                  for a in real.args], ["X", "W", "B"], ["Y"])
    monkeypatch.setattr(daceml_adapter, "mirror_expansion", lambda n, s, g: without_b)
    nsdfg = ns.donnx.ONNXConv.implementations["mi355x"].expansion(node, st, sdfg)
    (tasklet,) = [n for n in nsdfg.nodes()[0].nodes() if isinstance(n, _Tasklet)]
    assert sorted(tasklet.in_types) == ["_W", "_X"]
    assert sorted(e.dst_conn for e in nsdfg.nodes()[0].in_edges(tasklet)) == ["_W", "_X"]
    assert "B" in nsdfg.arrays   # still an argument of the nested SDFG, as the node's edge demands


def test_registered_expansion_falls_back_like_the_reference(fake_daceml):
    ns = fake_daceml
    daceml_adapter.register(["Softmax", "Conv"])
    # arrays in host memory: the kernels take device pointers, so the node goes to expand_node (onnx_op.py:668-680)
    soft = ns.donnx.ONNXSoftmax("host_sm", axis=-1)
    sdfg, st = _wire(soft, {"input": [4, 128]}, {"output": [4, 128]}, storage=light.StorageType.CPU_Heap)
    expansion = ns.donnx.ONNXSoftmax.implementations["mi355x"]
    assert expansion.forward_impl.forward_can_be_applied(soft, st, sdfg) is False
    assert expansion.expansion(soft, st, sdfg) == "onnxruntime-expansion"
    # a configuration the kernels refuse (grouped convolution) takes the same way out
    conv = ns.donnx.ONNXConv("grouped", group=2)
    sdfg, st = _wire(conv, {"X": [1, 4, 8, 8], "W": [4, 2, 3, 3]}, {"Y": [1, 4, 6, 6]})
    assert ns.donnx.ONNXConv.implementations["mi355x"].expansion(conv, st, sdfg) == "onnxruntime-expansion"
    assert ns.fallbacks == ["host_sm", "grouped"]
    # validation runs before anything else, as in the reference's Expansion.expansion
    bad = ns.donnx.ONNXSoftmax("bad", axis=-1)
    sdfg, st = _wire(bad, {}, {"output": [4, 128]})
    with pytest.raises(ValueError, match="missing 1 required input"):
        expansion.expansion(bad, st, sdfg)


def test_register_calls_post_parse_when_the_implementation_has_one(fake_daceml, monkeypatch):
    ns = fake_daceml
    daceml_adapter.register(["Softmax"])
    expansion = ns.donnx.ONNXSoftmax.implementations["mi355x"]
    seen = []
    monkeypatch.setattr(expansion.forward_impl, "post_parse", staticmethod(lambda n, s, g, r: seen.append((n.label, r))),
                        raising=False)
    soft = ns.donnx.ONNXSoftmax("pp", axis=-1)
    sdfg, st = _wire(soft, {"input": [2, 64]}, {"output": [2, 64]})
    result = expansion.expansion(soft, st, sdfg)
    assert seen == [("pp", result)]


def test_register_without_daceml_names_the_missing_package(monkeypatch):
    dace = types.ModuleType("dace")
    dace.library = types.ModuleType("dace.library")
    dace.transformation = types.ModuleType("dace.transformation")
    dace.transformation.transformation = types.ModuleType("dace.transformation.transformation")
    dace.transformation.transformation.ExpandTransformation = object
    for name, mod in {"dace": dace, "dace.library": dace.library, "dace.transformation": dace.transformation,
                      "dace.transformation.transformation": dace.transformation.transformation}.items():
        monkeypatch.setitem(sys.modules, name, mod)
    with pytest.raises(ImportError, match="daceml"):
        daceml_adapter.register()

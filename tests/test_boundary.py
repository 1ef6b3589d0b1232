"""Host-side tests that need no GPU: the C-ABI library loads and exports what the
header declares, the plugin registry and node classes behave like the
reference's, refusals are reported, and the ONNX reader/shape inference work."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest
import torch

import dace_onnx_amd as dml
from dace_onnx_amd import _lib, sdfg as dace
import dace_onnx_amd.onnx as donnx
from dace_onnx_amd.onnx import proto
from dace_onnx_amd.onnx.shape_inference import infer_shapes, ShapeInferenceError
from dace_onnx_amd.onnx.op_implementations.mi355x_implementations import _BatchPlan, _conv_geometry
from dace_onnx_amd.util import utils
from conftest import ROOT, GOLDEN_DIR


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mi355x_onnx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355x_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    declared = _declared_symbols()
    assert len(declared) >= 10
    lib = ctypes.CDLL(_lib.LIBRARY_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/mi355x_onnx.h but not exported"
    # the Python prototypes cover exactly the declared symbols
    assert sorted(_lib.SIGNATURES) == declared


def test_library_identity_and_error_channel():
    lib = _lib.library()
    assert lib.mi355x_version() == 100
    # argument validation happens on the host, before any launch: no GPU needed
    status = lib.mi355x_softmax_f32(None, None, -1, 4, 1, None)
    assert status == 1
    assert b"negative extent" in lib.mi355x_last_error()
    with pytest.raises(_lib.MI355XError, match="negative extent"):
        _lib.check(lib.mi355x_softmax_f32(None, None, -1, 4, 1, None), "softmax")
    assert lib.mi355x_eltwise_f32(99, None, None, None, 9, None, None, None, None) == 1
    assert b"ndim" in lib.mi355x_last_error()
    assert lib.mi355x_gemm_f32(None, None, None, None, None, 1, 1, 4, 4, 4, _lib.i64_array([0, 0, 4, 1]),
                               _lib.i64_array([0, 0, 4, 1]), _lib.i64_array([0, 0, 4]), None, 1.0, 64, None) == 1
    assert b"epilogue" in lib.mi355x_last_error()
    # empty problems are accepted and launch nothing
    assert lib.mi355x_softmax_f32(None, None, 0, 128, 1, None) == 0
    assert lib.mi355x_layernorm_f32(None, None, None, None, 0, 768, 1e-5, None) == 0
    assert lib.mi355x_matmul_integer_i8(None, None, None, None, None, 0, 16, 16, None) == 0


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIBRARY_PATH", os.path.join(ROOT, "does_not_exist.so"))
    with pytest.raises(_lib.LibraryNotBuilt):
        _lib.library()


# ----------------------------------------------------------------------------- registry / nodes
def test_registry_and_binding():
    impls = dict(donnx.ONNXForward.registered_implementations("Conv"))
    assert "mi355x" in impls
    for op in ("MatMul", "Gemm", "Conv", "MatMulInteger", "Softmax", "LayerNormalization", "Add", "Relu", "Gelu",
               "Transpose", "Reshape"):
        cls = donnx.get_onnx_node(op)
        assert {"mi355x", "onnxruntime"} <= set(cls.implementations), op
    assert donnx.has_onnx_node("MatMul") and not donnx.has_onnx_node("NonMaxSuppression")
    assert donnx.default_implementation == "mi355x"


def test_out_of_tree_implementation_is_selectable():
    calls = []

    @donnx.op_implementation(op="Relu", name="unit_test_impl")
    class MyRelu(donnx.ONNXForward):
        @staticmethod
        def forward_can_be_applied(node, state, sdfg):
            calls.append("can")
            return True

        @staticmethod
        def forward(node, state, sdfg):
            calls.append("fwd")
            return dace.KernelCall("k", "mi355x_eltwise_f32", [], ["X"], ["Y"])

    try:
        assert ":Implementation name: ``\"unit_test_impl\"``" in MyRelu.__doc__
        assert "unit_test_impl" in donnx.ONNXRelu.implementations
        sdfg = dace.SDFG("t")
        sdfg.add_array("a", [4], dace.float32)
        sdfg.add_array("b", [4], dace.float32)
        st = sdfg.add_state()
        n = donnx.ONNXRelu("r")
        n.implementation = "unit_test_impl"
        st.add_edge(st.add_read("a"), None, n, "X", sdfg.make_array_memlet("a"))
        st.add_edge(n, "Y", st.add_write("b"), None, sdfg.make_array_memlet("b"))
        sdfg.expand_library_nodes()
        assert calls == ["can", "fwd"]
    finally:
        donnx.ONNXRelu.implementations.pop("unit_test_impl")
        donnx.ONNXForward.unregister(MyRelu)


def test_node_construction_errors():
    n = donnx.ONNXConv("conv", strides=[2, 2])
    assert n.strides == [2, 2] and n.pads is None and n.group == 1 and n.auto_pad == "NOTSET"
    assert set(n.in_connectors) == {"X", "W"} and set(n.out_connectors) == {"Y"}  # optional B not pre-added
    with pytest.raises(TypeError, match="unexpected keyword argument 'foo'"):
        donnx.ONNXConv("conv", foo=3)
    with pytest.raises(TypeError, match="takes 1 positional"):
        donnx.ONNXConv("conv", 3)
    assert donnx.ONNXGemm("g").alpha == 1.0 and donnx.ONNXGemm("g").transB == 0
    assert donnx.ONNXSoftmax("s").axis == 1  # opset-11 default


def _one_node_sdfg(node, inputs, outputs):
    sdfg = dace.SDFG("t")
    st = sdfg.add_state()
    st.add_node(node)
    for conn, (shape, dtype) in inputs.items():
        sdfg.add_array("in_" + conn, shape, dtype)
        node.add_in_connector(conn)
        st.add_edge(st.add_read("in_" + conn), None, node, conn, sdfg.make_array_memlet("in_" + conn))
    for conn, (shape, dtype) in outputs.items():
        sdfg.add_array("out_" + conn, shape, dtype)
        node.add_out_connector(conn)
        st.add_edge(node, conn, st.add_write("out_" + conn), None, sdfg.make_array_memlet("out_" + conn))
    return sdfg, st


def test_validate_errors():
    f32, i8 = dace.float32, dace.int8
    sdfg, st = _one_node_sdfg(donnx.ONNXMatMul("m"), {"A": ([2, 3], f32)}, {"Y": ([2, 4], f32)})
    with pytest.raises(ValueError, match="MatMul missing 1 required input: 'B'"):
        sdfg.expand_library_nodes()
    sdfg, st = _one_node_sdfg(donnx.ONNXMatMul("m"), {"A": ([2, 3], f32), "B": ([3, 4], f32), "Q": ([1], f32)},
                              {"Y": ([2, 4], f32)})
    with pytest.raises(TypeError, match="unexpected argument 'Q'"):
        sdfg.expand_library_nodes()
    sdfg, st = _one_node_sdfg(donnx.ONNXMatMul("m"), {"A": ([2, 3], f32), "B": ([3, 4], dace.float64)},
                              {"Y": ([2, 4], f32)})
    with pytest.raises(ValueError, match="Could not solve type constraints"):
        sdfg.expand_library_nodes()
    sdfg, st = _one_node_sdfg(donnx.ONNXRelu("r"), {"X": ([4], i8)}, {"Y": ([4], i8)})
    with pytest.raises(ValueError, match="Expected type in"):
        sdfg.expand_library_nodes()


def test_validate_variadic_parameters_and_connectors():
    """The rest of the validation contract (onnx_op.py:197-415): variadic connectors are numbered 0..n-1 without
    gaps, `__` belongs to variadic parameters only, every edge ends on a declared connector, required attributes
    are set, and the edges come back in schema order whatever order they were added in."""
    f32 = dace.float32
    ok = {"data_0__1": ([4], f32), "data_0__0": ([4], f32), "data_0__2": ([4], f32)}
    node = donnx.ONNXSum("s")
    sdfg, st = _one_node_sdfg(node, ok, {"sum": ([4], f32)})
    node.validate(sdfg, st)
    assert [e.dst_conn for e in node.iter_inputs_in_onnx_order(st)] == ["data_0__0", "data_0__1", "data_0__2"]
    assert [(e.dst_conn if i else e.src_conn) for e, i in node.iter_edges(st)] == ["data_0__0", "data_0__1", "data_0__2", "sum"]
    node = donnx.ONNXSum("s")
    sdfg, st = _one_node_sdfg(node, {"data_0__0": ([4], f32), "data_0__2": ([4], f32)}, {"sum": ([4], f32)})
    with pytest.raises(ValueError, match="expected variadic parameter with number 1"):
        node.validate(sdfg, st)
    node = donnx.ONNXSum("s")
    sdfg, st = _one_node_sdfg(node, {"data_0__0": ([4], f32), "other__1": ([4], f32)}, {"sum": ([4], f32)})
    with pytest.raises(ValueError, match="unexpected variadic argument 'other__1'"):
        node.validate(sdfg, st)
    node = donnx.ONNXSum("s")
    sdfg, st = _one_node_sdfg(node, {"data_0__00": ([4], f32)}, {"sum": ([4], f32)})
    with pytest.raises(ValueError, match="leading zeroes"):
        node.validate(sdfg, st)
    node = donnx.ONNXRelu("r")
    sdfg, st = _one_node_sdfg(node, {"X__0": ([4], f32)}, {"Y": ([4], f32)})
    with pytest.raises(ValueError, match="non-variadic parameter 'X'"):
        node.validate(sdfg, st)
    # an edge on a connector the node does not declare
    node = donnx.ONNXConv("c")
    sdfg, st = _one_node_sdfg(node, {"X": ([1, 1, 4, 4], f32), "W": ([1, 1, 3, 3], f32), "B": ([1], f32)}, {"Y": ([1, 1, 2, 2], f32)})
    node.validate(sdfg, st)
    node.remove_in_connector("B")
    with pytest.raises(ValueError, match="nonexistent input connector 'B'"):
        node.validate(sdfg, st)
    # inputs in schema order although W was connected before X
    node = donnx.ONNXConv("c")
    sdfg, st = _one_node_sdfg(node, {"W": ([1, 1, 3, 3], f32), "X": ([1, 1, 4, 4], f32)}, {"Y": ([1, 1, 2, 2], f32)})
    assert [e.dst_conn for e in node.iter_inputs_in_onnx_order(st)] == ["X", "W"]
    # missing output, several missing inputs
    node = donnx.ONNXGemm("g")
    sdfg, st = _one_node_sdfg(node, {}, {"Y": ([2, 2], f32)})
    with pytest.raises(ValueError, match="Gemm missing 2 required inputs: 'A', and 'B'"):
        node.validate(sdfg, st)
    node = donnx.ONNXRelu("r")
    sdfg, st = _one_node_sdfg(node, {"X": ([4], f32)}, {})
    with pytest.raises(ValueError, match="Relu missing 1 required output: 'Y'"):
        node.validate(sdfg, st)
    # a required attribute left unset
    node = donnx.ONNXCast("c", to=1)
    node.to = None
    sdfg, st = _one_node_sdfg(node, {"input": ([4], f32)}, {"output": ([4], f32)})
    with pytest.raises(ValueError, match="required attribute 'to'"):
        node.validate(sdfg, st)
    with pytest.raises(TypeError, match="missing 1 required keyword-only argument: 'to'"):
        donnx.ONNXCast("c")


@pytest.mark.parametrize("case", ["matmul_1d", "conv_group", "conv_3d", "mmi_zp_wrong_length", "gelu_tanh", "ln_mean_out",
                                  "softmax_f64", "gemm_beta"])
def test_refusal_is_an_error_not_a_fallback(case):
    """forward_can_be_applied -> False falls back to "onnxruntime" (onnx_op.py:668-680), which this
    build does not have: the expansion must raise instead of computing anywhere else."""
    f32, i8, i32 = dace.float32, dace.int8, dace.int32
    if case == "matmul_1d":  # PureMatMul refuses 1-D operands as well (:133-140)
        sdfg, _ = _one_node_sdfg(donnx.ONNXMatMul("m"), {"A": ([3], f32), "B": ([3, 4], f32)}, {"Y": ([4], f32)})
    elif case == "conv_group":
        sdfg, _ = _one_node_sdfg(donnx.ONNXConv("c", group=2), {"X": ([1, 4, 8, 8], f32), "W": ([4, 2, 3, 3], f32)},
                                 {"Y": ([1, 4, 6, 6], f32)})
    elif case == "conv_3d":
        sdfg, _ = _one_node_sdfg(donnx.ONNXConv("c"), {"X": ([1, 2, 8, 8, 8], f32), "W": ([4, 2, 3, 3, 3], f32)},
                                 {"Y": ([1, 4, 6, 6, 6], f32)})
    elif case == "mmi_zp_wrong_length":
        sdfg, _ = _one_node_sdfg(donnx.ONNXMatMulInteger("m"),
                                 {"A": ([4, 8], i8), "B": ([8, 4], i8), "a_zero_point": ([3], i8)}, {"Y": ([4, 4], i32)})
    elif case == "gelu_tanh":
        sdfg, _ = _one_node_sdfg(donnx.ONNXGelu("g", approximate="tanh"), {"X": ([4], f32)}, {"Y": ([4], f32)})
    elif case == "ln_mean_out":
        sdfg, _ = _one_node_sdfg(donnx.ONNXLayerNormalization("l"), {"X": ([4, 8], f32), "Scale": ([8], f32)},
                                 {"Y": ([4, 8], f32), "Mean": ([4, 1], f32)})
    elif case == "softmax_f64":
        sdfg, _ = _one_node_sdfg(donnx.ONNXSoftmax("s"), {"input": ([4, 8], dace.float64)},
                                 {"output": ([4, 8], dace.float64)})
    else:
        sdfg, _ = _one_node_sdfg(donnx.ONNXGemm("g", beta=0.5), {"A": ([4, 8], f32), "B": ([8, 4], f32), "C": ([4], f32)},
                                 {"Y": ([4, 4], f32)})
    with pytest.raises(donnx.ExpansionRefused, match="onnxruntime"):
        sdfg.expand_library_nodes()


def test_unexpanded_graph_cannot_run():
    sdfg, _ = _one_node_sdfg(donnx.ONNXRelu("r"), {"X": ([4], dace.float32)}, {"Y": ([4], dace.float32)})
    with pytest.raises(RuntimeError, match="not expanded"):
        dace.CompiledSDFG(sdfg)


def test_matmul_expansion_folds_batch_into_m_and_emits_cpp():
    sdfg, st = _one_node_sdfg(donnx.ONNXMatMul("Matmul"), {"A": ([8, 128, 768], dace.float32),
                                                           "B": ([768, 3072], dace.float32)},
                              {"Y": ([8, 128, 3072], dace.float32)})
    utils.expand_onnx_nodes(sdfg)
    calls = [n for n, _ in sdfg.all_nodes_recursive() if isinstance(n, dace.KernelCall)]
    assert len(calls) == 1 and calls[0].function == "mi355x_gemm_f32"
    args = calls[0].args
    assert args[5:10] == [1, 1, 1024, 3072, 768]  # batch folded into M
    cpp = calls[0].as_cpp()
    assert "mi355x_gemm_f32(_A, _B, _Y, nullptr, nullptr, 1, 1, 1024, 3072, 768" in cpp
    assert "__dace_current_stream" in cpp


def test_batch_plan_attention_shapes():
    f = dace.float32
    q = dace.Array(f, [8, 12, 128, 64])
    kt = dace.Array(f, [8, 12, 64, 128], strides=[98304, 8192, 1, 64])  # K^T as a strided view
    y = dace.Array(f, [8, 12, 128, 128])
    p = _BatchPlan(q, kt, y)
    assert p.ok and (p.batch0 * p.batch1, p.M, p.N, p.K) == (96, 128, 128, 64)
    assert p.b_strides[2:] == [1, 64]
    # head-split view of a [8,128,768] projection: two real batch levels
    qv = dace.Array(f, [8, 12, 128, 64], strides=[98304, 64, 768, 1])
    p = _BatchPlan(qv, kt, y)
    assert p.ok and (p.batch0, p.batch1) == (8, 12) and p.a_strides == [98304, 64, 768, 1]
    # broadcast B over a 3-level batch that cannot be merged -> refused
    a5 = dace.Array(f, [2, 3, 4, 5, 6], strides=[1000, 200, 40, 6, 1])
    b2 = dace.Array(f, [6, 7])
    assert not _BatchPlan(a5, b2, dace.Array(f, [2, 3, 4, 5, 7])).ok


def test_conv_geometry_auto_pad():
    n = donnx.ONNXConv("c", auto_pad="SAME_UPPER", strides=[2, 2])
    X, W = dace.Array(dace.float32, [1, 3, 7, 8]), dace.Array(dace.float32, [4, 3, 3, 3])
    pads, strides, dil, oh, ow = _conv_geometry(n, X, W)
    assert (oh, ow) == (4, 4) and pads == [1, 0, 1, 1]
    n = donnx.ONNXConv("c", pads=[1, 1, 1, 1])
    assert _conv_geometry(n, X, W)[3:] == (7, 8)
    assert _conv_geometry(donnx.ONNXConv("c", kernel_shape=[5, 5]), X, W) is None


# ----------------------------------------------------------------------------- ONNX files
def test_proto_reads_reference_fixture():
    # data fixture of the reference's own tests (tests/onnx_files/slice.onnx)
    m = proto.load(os.path.join(GOLDEN_DIR, "slice.onnx"))
    assert [o.version for o in m.opset_import] == [12]
    (node, ) = m.graph.node
    assert node.op_type == "Slice" and node.input == ["data", "starts", "ends", "axes"] and node.output == ["output"]
    assert [(t.name, t.array.tolist()) for t in m.graph.initializer] == [("starts", [0]), ("ends", [1]), ("axes", [0])]
    assert m.graph.input[0].shape == [2] and m.graph.output[0].shape == [1]
    data = open(os.path.join(GOLDEN_DIR, "slice.onnx"), "rb").read()
    assert proto.serialize_model(proto.parse_model(proto.serialize_model(m))) == proto.serialize_model(m)
    assert len(proto.serialize_model(m)) in (len(data), len(data) + 2)  # producer_name field is written empty
    model = donnx.ONNXModel("slice", m, fold_constants=False)       # imports and expands without a GPU
    calls = [n for n, _ in model.expand().all_nodes_recursive() if isinstance(n, dace.KernelCall)]
    assert [c.function for c in calls] == ["mi355x_permute_b32"] and calls[0].args[3].values == [1]
    with pytest.raises(ValueError, match="Unsupported ONNX operator: 'NonZero'"):
        bad = proto.parse_model(proto.serialize_model(m))
        bad.graph.node[0].op_type = "NonZero"
        donnx.ONNXModel("nonzero", bad)


def test_reference_bert_subgraph_fixture_imports_and_folds():
    """tests/onnx_files/reshape.onnx of the reference (Slice of the position embeddings, Cast of the target
    shape, Reshape): imported as in tests/test_bert_subgraphs.py:29-32 with fold_constants=False -- the Reshape
    target is then computed by the Cast node and the result's shape comes from the model's declaration -- and
    with folding, which (tests/transformation/test_constant_folding.py:17-41) leaves only the data path."""
    m = proto.load(os.path.join(GOLDEN_DIR, "reshape.onnx"))
    assert [n.op_type for n in m.graph.node] == ["Slice", "Cast", "Reshape"] and not m.graph.input
    unfolded = donnx.ONNXModel("bert_subgraph", m, fold_constants=False, fuse=False)
    calls = [n.function for n, _ in unfolded.expand().all_nodes_recursive() if isinstance(n, dace.KernelCall)]
    assert sorted(calls) == ["mi355x_cast", "mi355x_permute_b32"]
    folded = donnx.ONNXModel("bert_subgraph_folded", m, fold_constants=True, fuse=False)
    calls = [n.function for n, _ in folded.expand().all_nodes_recursive() if isinstance(n, dace.KernelCall)]
    assert calls == []       # the Slice of a constant folds, the Cast folds, the Reshape is a view


def test_proto_roundtrip_all_attribute_kinds():
    t = proto.numpy_helper.from_array(np.arange(6, dtype=np.int64).reshape(2, 3) - 3, "t")
    node = proto.helper.make_node("Conv", ["X", "W", ""], ["Y"], name="n", pads=[1, 2, 3, 4], auto_pad="NOTSET",
                                  alpha=0.25, group=-1, scales=[0.5, 1.5], value=t, names=["a", "b"])
    g = proto.helper.make_graph([node], "g", [proto.helper.make_tensor_value_info("X", proto.TensorProto.FLOAT, [1, "N", 3])],
                                [proto.helper.make_tensor_value_info("Y", proto.TensorProto.INT8, None)],
                                initializer=[proto.numpy_helper.from_array(np.float32([[1.5, -2.0]]), "W")])
    m2 = proto.parse_model(proto.serialize_model(proto.helper.make_model(g)))
    n2 = m2.graph.node[0]
    attrs = {a.name: a.value for a in n2.attribute}
    assert n2.input == ["X", "W", ""] and attrs["pads"] == [1, 2, 3, 4] and attrs["auto_pad"] == "NOTSET"
    assert attrs["alpha"] == 0.25 and attrs["group"] == -1 and attrs["scales"] == [0.5, 1.5] and attrs["names"] == ["a", "b"]
    assert np.array_equal(attrs["value"].array, t.array) and attrs["value"].array.dtype == np.int64
    assert m2.graph.input[0].shape == [1, "N", 3] and m2.graph.output[0].shape is None
    assert m2.graph.output[0].elem_type == proto.TensorProto.INT8
    assert np.array_equal(m2.graph.initializer[0].array, np.float32([[1.5, -2.0]]))


def test_shape_inference_bert_layer_graph():
    from dace_onnx_amd.testing.graphs import bert_encoder_layer_model
    from oracle import pure_ops
    w = pure_ops.bert_layer_weights(np.random.default_rng(0), hidden=64, ffn=128)
    m = infer_shapes(bert_encoder_layer_model(w, 2, 16, 4))
    shapes = {v.name: v.shape for v in m.graph.value_info}
    assert shapes["q_heads"] == [2, 4, 16, 16] and shapes["k_t"] == [2, 4, 16, 16]
    assert shapes["scores"] == [2, 4, 16, 16] and shapes["ctx"] == [2, 16, 64] and shapes["inter"] == [2, 16, 128]
    bad = proto.helper.make_graph([proto.helper.make_node("MatMul", ["a", "b"], ["c"])], "g",
                                  [proto.helper.make_tensor_value_info("a", 1, [2, 3]),
                                   proto.helper.make_tensor_value_info("b", 1, [4, 5])],
                                  [proto.helper.make_tensor_value_info("c", 1, None)])
    with pytest.raises(ShapeInferenceError, match="inner dimensions"):
        infer_shapes(proto.helper.make_model(bad))


def test_clean_onnx_name_table():
    from dace_onnx_amd.onnx.onnx_importer import clean_onnx_name
    # daceml/onnx/converters.py:204-211
    assert clean_onnx_name("bert/embeddings/Reshape_4:0") == "bertSLASHembeddingsSLASHReshape_4COLON0"
    assert clean_onnx_name("0.weight-x") == "ONNX_0DOTweightDASHx"


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "dace-onnx_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(base, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), os.path.join(base, f)


def test_daceml_adapter_mirrors_nodes_and_needs_the_real_packages():
    from dace_onnx_amd import daceml_adapter
    # the mirror runs on anything with the SDFG attribute surface; on this package's own objects it must
    # reproduce the direct expansion (same C++ tasklet text)
    node = donnx.ONNXMatMul("Matmul")
    sdfg, st = _one_node_sdfg(node, {"A": ([8, 128, 768], dace.float32), "B": ([768, 3072], dace.float32)},
                              {"Y": ([8, 128, 3072], dace.float32)})
    call = daceml_adapter.mirror_expansion(node, st, sdfg)
    assert call.function == "mi355x_gemm_f32"
    assert "mi355x_gemm_f32(_A, _B, _Y, nullptr, nullptr, 1, 1, 1024, 3072, 768" in call.as_cpp()
    conv = donnx.ONNXConv("Conv", strides=[2, 2])
    sdfg, st = _one_node_sdfg(conv, {"X": ([5, 3, 10, 10], dace.float32), "W": ([16, 3, 3, 3], dace.float32)},
                              {"Y": ([5, 16, 4, 4], dace.float32)})
    cpp = daceml_adapter.mirror_expansion(conv, st, sdfg).as_cpp()
    assert "mi355x_conv2d_f32(_X, _W, nullptr, _Y, 5, 3, 10, 10, 16, 3, 3" in cpp and "__dace_current_stream" in cpp
    # a node the implementation refuses (1-D operand) mirrors to None: the adapter then falls back like the reference
    mm = donnx.ONNXMatMul("Matmul1d")
    sdfg, st = _one_node_sdfg(mm, {"A": ([4], dace.float32), "B": ([4, 3], dace.float32)}, {"Y": ([3], dace.float32)})
    assert daceml_adapter.mirror_expansion(mm, st, sdfg) is None
    with pytest.raises(ImportError, match="dace"):
        daceml_adapter.register()


def test_onnx_model_helpers_of_the_reference_api():
    # ONNXModel.expand_onnx_nodes (expansion without fusion) and create_output_array (onnx_importer.py:574-633)
    from dace_onnx_amd.onnx.onnx_importer import create_output_array
    from dace_onnx_amd.testing.graphs import conv_relu_model
    rng = np.random.default_rng(0)
    m = conv_relu_model(rng.normal(size=(4, 3, 3, 3)).astype(np.float32), np.zeros(4, np.float32), (1, 3, 8, 8))
    model = donnx.ONNXModel("conv_relu_unfused", m)
    model.expand_onnx_nodes()
    fns = [n.function for n, _ in model.sdfg.all_nodes_recursive() if isinstance(n, dace.KernelCall)]
    assert fns == ["mi355x_conv2d_f32", "mi355x_eltwise_f32"]      # Relu not folded into the convolution
    desc = model.sdfg.arrays["Y"]
    out = create_output_array({}, desc, use_torch=True, zeros=True)
    assert tuple(out.shape) == tuple(desc.shape) and out.dtype == torch.float32 and float(out.abs().sum()) == 0.0
    with pytest.raises(ValueError, match="use_torch=False"):
        create_output_array({}, desc, use_torch=False)


def test_trace_build_is_separate_from_the_library(monkeypatch, tmp_path):
    """The workgroup trace lives in a second build (`make trace`): the script that reads it asks for that file by name and
    says how to build it when it is missing; the product library exports no trace symbol."""
    from dace_onnx_amd.testing import wg_trace
    assert os.path.basename(wg_trace.TRACE_LIBRARY) == "libmi355x_onnx_trace.so"
    assert os.path.dirname(wg_trace.TRACE_LIBRARY) == os.path.dirname(_lib.LIBRARY_PATH)
    monkeypatch.setattr(wg_trace, "TRACE_LIBRARY", str(tmp_path / "absent.so"))
    with pytest.raises(_lib.LibraryNotBuilt, match="make -C dace-onnx_amd/csrc trace"):
        wg_trace.load_trace_library()
    exported = subprocess.run(["nm", "-D", "--defined-only", _lib.LIBRARY_PATH], capture_output=True, text=True, check=True).stdout
    assert "trace_buffer" not in exported

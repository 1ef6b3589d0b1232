"""Constant folding at import (reference: daceml/transformation/constant_folding.py, applied by
ONNXModel when fold_constants is set): each rule against numpy on hand-built graphs, and the chain the
TorchScript exporter writes for a Reshape target."""
import numpy as np
import pytest

import dace_onnx_amd.onnx as donnx
from dace_onnx_amd.onnx import proto
from dace_onnx_amd.transformation.constant_folding import fold_constants, MAX_FOLDED_VIEW_ELEMENTS

H, T = proto.helper, proto.TensorProto


def _fold(nodes, inits, out_name, inputs=()):
    g = H.make_graph(nodes, "g", list(inputs), [H.make_tensor_value_info(out_name, T.FLOAT, None)],
                     initializer=[proto.numpy_helper.from_array(v, name=k) for k, v in inits.items()])
    m = fold_constants(H.make_model(g, opset_imports=[H.make_opsetid("", 12)]))
    return m, {t.name: np.asarray(t.array).reshape(t.dims) for t in m.graph.initializer}


def test_exporters_reshape_target_chain():
    # Constant(2) -> Unsqueeze, Constant(128) -> Unsqueeze, Constant(-1) ..., Concat -> Reshape target
    inits = {"b": np.array(2, np.int64), "s": np.array(128, np.int64), "m1": np.array(-1, np.int64),
             "d": np.array(64, np.int64)}
    nodes = [H.make_node("Unsqueeze", [k], [k + "_u"], axes=[0]) for k in inits]
    nodes.append(H.make_node("Concat", [k + "_u" for k in inits], ["target"], axis=0))
    nodes.append(H.make_node("Reshape", ["x", "target"], ["y"]))
    m, consts = _fold(nodes, inits, "y", inputs=[H.make_tensor_value_info("x", T.FLOAT, [2, 128, 128])])
    assert [n.op_type for n in m.graph.node] == ["Reshape"]
    assert consts["target"].tolist() == [2, 128, -1, 64] and consts["target"].dtype == np.int64
    assert set(consts) == {"target"}       # the scalars nothing reads any more are gone


@pytest.mark.parametrize("case", ["shape_gather", "slice_cast", "arith", "squeeze_neg", "constant_of_shape_range"])
def test_rules(case):
    x_info = H.make_tensor_value_info("x", T.FLOAT, [4, 6, 10])
    if case == "shape_gather":
        nodes = [H.make_node("Shape", ["x"], ["s"]), H.make_node("Gather", ["s", "i"], ["g"], axis=0),
                 H.make_node("Unsqueeze", ["g"], ["gu"], axes=[-1]), H.make_node("Concat", ["gu", "m"], ["t"], axis=0),
                 H.make_node("Reshape", ["x", "t"], ["y"])]
        m, c = _fold(nodes, {"i": np.array(0, np.int64), "m": np.array([-1], np.int64)}, "y", inputs=[x_info])
        assert [n.op_type for n in m.graph.node] == ["Reshape"] and c["t"].tolist() == [4, -1]
    elif case == "slice_cast":
        nodes = [H.make_node("Shape", ["x"], ["s"]),
                 H.make_node("Slice", ["s", "st", "en", "ax", "sp"], ["sl"]),
                 H.make_node("Cast", ["sl"], ["f"], to=T.FLOAT), H.make_node("Mul", ["x", "f"], ["y"])]
        m, c = _fold(nodes, {"st": np.array([2], np.int64), "en": np.array([100], np.int64), "ax": np.array([0], np.int64),
                             "sp": np.array([1], np.int64)}, "y", inputs=[x_info])
        assert [n.op_type for n in m.graph.node] == ["Mul"]
        assert c["f"].dtype == np.float32 and c["f"].tolist() == [10.0]
    elif case == "arith":
        nodes = [H.make_node("Add", ["a", "b"], ["ab"]), H.make_node("Div", ["ab", "two"], ["q"]),
                 H.make_node("Sub", ["q", "b"], ["d"]), H.make_node("Mul", ["d", "d"], ["sq"]),
                 H.make_node("Reshape", ["x", "sq"], ["y"])]
        m, c = _fold(nodes, {"a": np.array([-7, 9], np.int64), "b": np.array([2, 2], np.int64),
                             "two": np.array(2, np.int64)}, "y", inputs=[x_info])
        # (-7 + 2) / 2 truncates toward zero: -2, not -3
        assert c["sq"].tolist() == [16, 9] and [n.op_type for n in m.graph.node] == ["Reshape"]
    elif case == "squeeze_neg":
        nodes = [H.make_node("Squeeze", ["a"], ["s"], axes=[0]), H.make_node("Neg", ["s"], ["n"]),
                 H.make_node("Sqrt", ["p"], ["r"]), H.make_node("Identity", ["r"], ["ri"]),
                 H.make_node("Mul", ["x", "ri"], ["y0"]), H.make_node("Add", ["y0", "n"], ["y"])]
        m, c = _fold(nodes, {"a": np.array([[1.0, 2.0]], np.float32), "p": np.array(16.0, np.float32)}, "y", inputs=[x_info])
        assert [n.op_type for n in m.graph.node] == ["Mul", "Add"]
        assert c["n"].tolist() == [-1.0, -2.0] and c["ri"].item() == 4.0
    else:
        nodes = [H.make_node("ConstantOfShape", ["sh"], ["z"], value=proto.numpy_helper.from_array(np.array([3], np.int64))),
                 H.make_node("Range", ["r0", "r1", "r2"], ["r"]), H.make_node("Add", ["z", "r"], ["t"]),
                 H.make_node("Reshape", ["x", "t"], ["y"])]
        m, c = _fold(nodes, {"sh": np.array([3], np.int64), "r0": np.array(1, np.int64), "r1": np.array(7, np.int64),
                             "r2": np.array(2, np.int64)}, "y", inputs=[x_info])
        assert c["t"].tolist() == [4, 6, 8]


def test_large_weight_transpose_stays_a_node_and_unknown_ops_are_left_alone():
    w = np.zeros((128, 64), np.float32)
    assert w.size > MAX_FOLDED_VIEW_ELEMENTS
    nodes = [H.make_node("Transpose", ["w"], ["wt"], perm=[1, 0]), H.make_node("MatMul", ["x", "wt"], ["h"]),
             H.make_node("Transpose", ["small"], ["small_t"], perm=[1, 0]), H.make_node("Erf", ["small_t"], ["e"]),
             H.make_node("Add", ["h", "e"], ["y"])]
    m, c = _fold(nodes, {"w": w, "small": np.arange(6, dtype=np.float32).reshape(2, 3)}, "y",
                 inputs=[H.make_tensor_value_info("x", T.FLOAT, [4, 64])])
    assert [n.op_type for n in m.graph.node] == ["Transpose", "MatMul", "Erf", "Add"]   # Erf has no folding rule
    assert c["small_t"].shape == (3, 2) and "wt" not in c


def test_model_without_constant_subgraphs_is_returned_as_is_and_switch_is_honoured():
    nodes = [H.make_node("Unsqueeze", ["c"], ["cu"], axes=[0]), H.make_node("Add", ["x", "cu"], ["y"])]
    g = H.make_graph(nodes, "g", [H.make_tensor_value_info("x", T.FLOAT, [2, 3])],
                     [H.make_tensor_value_info("y", T.FLOAT, [2, 3])],
                     initializer=[proto.numpy_helper.from_array(np.ones(3, np.float32), name="c")])
    model = H.make_model(g, opset_imports=[H.make_opsetid("", 12)])
    plain = H.make_model(H.make_graph(nodes[1:], "g", g.input, g.output,
                                      initializer=[proto.numpy_helper.from_array(np.ones((1, 3), np.float32), name="cu")]),
                         opset_imports=[H.make_opsetid("", 12)])
    assert fold_constants(plain) is plain
    folded = donnx.ONNXModel("folded", model)
    assert "cu" in folded.weights and len(model.graph.node) == 2      # caller's model untouched
    # with the switch off the Unsqueeze stays a node of the graph (a view at run time)
    kept = donnx.ONNXModel("not_folded", model, fold_constants=False)
    assert "cu" not in kept.weights and any(type(n).__name__ == "ONNXUnsqueeze" for n, _ in kept.sdfg.all_nodes_recursive())

"""A BertLayer as `torch.onnx.export(opset_version=12)` really writes it
(tests/golden/make_bert_layer_export.py): the hand-written ONNX reader, the importer's handling of
Constant nodes (reference: daceml/onnx/onnx_importer.py:193-229), the fusion pass on the exporter's own
node list, and -- on the GPU -- the result against the output PyTorch computed for the same input."""
import collections
import os

import numpy as np
import pytest

from dace_onnx_amd import sdfg as dace
import dace_onnx_amd.onnx as donnx
from dace_onnx_amd.onnx import proto
from conftest import GOLDEN_DIR, rel_err, FP32_REL_TOL

ONNX_FILE = os.path.join(GOLDEN_DIR, "bert_layer_torch_export_opset12.onnx")
H = proto.helper


def _launches(model):
    return [n.function for n, _ in model.expand().all_nodes_recursive() if isinstance(n, dace.KernelCall)]


def test_reader_parses_the_exporters_file():
    m = proto.load(ONNX_FILE)
    assert [(o.domain, o.version) for o in m.opset_import] == [("", 12)]
    assert [i.name for i in m.graph.input] == ["hidden_states"] and [o.name for o in m.graph.output] == ["output"]
    ops = collections.Counter(n.op_type for n in m.graph.node)
    # the decomposed forms the reference executes node by node: LayerNorm as ReduceMean/Sub/Pow/.../Sqrt/Div,
    # Gelu through Erf, the head split as Reshape/Transpose with Constant shapes
    assert ops == {"Add": 13, "Constant": 12, "Div": 3, "Erf": 1, "MatMul": 8, "Mul": 5, "Pow": 2, "ReduceMean": 4,
                   "Reshape": 4, "Softmax": 1, "Sqrt": 2, "Sub": 2, "Transpose": 4}
    weights = {t.name: tuple(t.dims) for t in m.graph.initializer}
    assert weights["attention.self.query.bias"] == (128, ) and weights["intermediate.dense.bias"] == (256, )
    assert sorted(d for d in weights.values() if len(d) == 2) == [(128, 128)] * 4 + [(128, 256), (256, 128)]
    # a round trip through the writer is byte-stable from the second pass on
    again = proto.serialize_model(proto.parse_model(proto.serialize_model(m)))
    assert again == proto.serialize_model(m)


def test_constant_nodes_become_weights():
    m = proto.load(ONNX_FILE)
    model = donnx.ONNXModel("torch_export", m, auto_optimize=False)
    state = model.sdfg.states()[0]
    assert not any(type(n).__name__ == "ONNXConstant" for n in state.nodes())
    constants = [n.output[0] for n in m.graph.node if n.op_type == "Constant"]
    assert len(constants) == 12 and all(c in model.weights for c in constants)
    shapes = sorted(tuple(model.weights[c].tolist()) for c in constants if model.weights[c].dim() == 1)
    assert shapes == [(2, 128, -1), (2, 128, -1, 64), (2, 128, -1, 64), (2, 128, -1, 64)]   # Reshape targets: head merge, head split x3
    assert sum(n.op_type == "Constant" for n in m.graph.node) == 12   # the caller's model is left as it was


def test_constant_node_checks():
    def model(node):
        g = H.make_graph([node, H.make_node("Relu", ["c"], ["y"])], "g", [],
                         [H.make_tensor_value_info("y", proto.TensorProto.FLOAT, [2])])
        return H.make_model(g, opset_imports=[H.make_opsetid("", 12)])

    value = proto.numpy_helper.from_array(np.array([1.0, -2.0], np.float32))
    ok = donnx.ONNXModel("c_ok", model(H.make_node("Constant", [], ["c"], value=value)))
    assert np.array_equal(ok.weights["c"].cpu().numpy(), [1.0, -2.0])
    with pytest.raises(ValueError, match="exactly one of its attributes"):
        donnx.ONNXModel("c_two", model(H.make_node("Constant", [], ["c"], value=value, value_float=1.0)))
    with pytest.raises(ValueError, match="unexpected attributes"):
        donnx.ONNXModel("c_attr", model(H.make_node("Constant", [], ["c"], axis=1)))
    with pytest.raises(ValueError, match="no inputs and exactly 1 output"):
        donnx.ONNXModel("c_in", model(H.make_node("Constant", ["y"], ["c"], value=value)))


def test_exported_layer_fuses_to_seven_launches():
    fused = _launches(donnx.ONNXModel("torch_export_fused", ONNX_FILE))
    assert sorted(fused) == sorted(["mi355x_gemm_f32"] * 4 + ["mi355x_attention_f32"] + ["mi355x_layernorm_f32"] * 2)
    unfused = _launches(donnx.ONNXModel("torch_export_unfused", ONNX_FILE, fuse=False))
    assert len(unfused) == 49 - 4     # every node but the 12 Constants; the 4 Reshapes are views
    assert unfused.count("mi355x_gemm_f32") == 8 and unfused.count("mi355x_reduce_mean_f32") == 4


@pytest.mark.gpu
@pytest.mark.parametrize("fuse,hip_graph", [(True, False), (True, True), (False, False)])
def test_exported_layer_matches_pytorch(fuse, hip_graph):
    ref = np.load(os.path.join(GOLDEN_DIR, "bert_layer_torch_export_opset12.npz"))
    model = donnx.ONNXModel(f"torch_export_{int(fuse)}{int(hip_graph)}", ONNX_FILE, fuse=fuse, use_hip_graph=hip_graph)
    for _ in range(3 if hip_graph else 1):      # replays after the capture as well
        out = model(ref["hidden_states"])
        assert rel_err(ref["output"], out) < FP32_REL_TOL

"""Graph-level fusion pass, checked without a GPU: the model is imported, fused and
expanded to kernel calls on the host, and the launch list is inspected."""
import numpy as np
import pytest

from dace_onnx_amd import sdfg as dace
import dace_onnx_amd.onnx as donnx
from dace_onnx_amd.onnx import proto
from dace_onnx_amd.testing.graphs import bert_encoder_layer_model
from dace_onnx_amd.transformation.fusion import _rebase_strides, _reshape_strides
from oracle import pure_ops

H = proto.helper


def _launches(model):
    sdfg = model.expand()
    out = []
    for n, _ in sdfg.all_nodes_recursive():
        if isinstance(n, dace.KernelCall):
            out.append((n.function, [a.values if isinstance(a, dace.I64Array) else a for a in n.args]))
    return out


def _bert(fuse):
    w = pure_ops.bert_layer_weights(np.random.default_rng(0), hidden=64, ffn=128)
    return donnx.ONNXModel("bert_small", bert_encoder_layer_model(w, 2, 16, 4), fuse=fuse)


def test_unfused_bert_layer_launches_every_node():
    names = [f for f, _ in _launches(_bert(False))]
    assert names.count("mi355x_gemm_f32") == 8 and names.count("mi355x_permute_b32") == 5
    assert len(names) == 26


def test_fused_bert_layer_is_nine_launches():
    calls = _launches(_bert(True))
    assert [f for f, _ in calls] == ["mi355x_gemm_f32"] * 2 + ["mi355x_softmax_f32"] + ["mi355x_gemm_f32"] * 2 + \
        ["mi355x_layernorm_f32"] + ["mi355x_gemm_f32"] * 2 + ["mi355x_layernorm_f32"]
    qkv, scores, _, ctx, out, _, ffn1, ffn2, _ = [a for _, a in calls]
    # Q, K, V projections: one GEMM of width 3 * 64 with the concatenated bias, weight k-contiguous
    assert qkv[5:10] == [1, 1, 32, 192, 64] and qkv[11] == [0, 0, 1, 64] and qkv[15] == 1
    # Q K^T reads Q at column 0 and K at column 64 of the wide result, scaled by 1/sqrt(16)
    assert (scores[0].offset, scores[1].offset) == (0, 64)
    assert scores[5:10] == [2, 4, 16, 16, 16]
    assert scores[10] == [16 * 192, 16, 192, 1] and scores[11] == [16 * 192, 16, 1, 192]
    assert scores[14] == pytest.approx(0.25)
    # P V reads V at column 128 and writes heads merged: [B, S, H * D]
    assert ctx[1].offset == 128 and ctx[11] == [16 * 192, 16, 192, 1] and ctx[12] == [16 * 64, 16, 64]
    # output projection and FFN: bias (1), Gelu (4), residual (8) in the epilogue
    assert out[15] == 9 and ffn1[15] == 5 and ffn2[15] == 9


def test_bert_base_attention_core_is_one_launch():
    # 128 keys, head size 64: MatMul -> Div -> Softmax -> MatMul becomes the fused attention kernel, which reads
    # Q, K, V as column slices of the wide projection and writes the heads merged
    w = pure_ops.bert_layer_weights(np.random.default_rng(0), hidden=768, ffn=3072)
    calls = _launches(donnx.ONNXModel("bert_base", bert_encoder_layer_model(w, 2, 128, 12)))
    assert sorted(f for f, _ in calls) == ["mi355x_attention_f32"] + ["mi355x_gemm_f32"] * 4 + ["mi355x_layernorm_f32"] * 2
    a = [args for f, args in calls if f == "mi355x_attention_f32"][0]
    assert [x.offset for x in a[:4]] == [0, 768, 1536, 0]
    assert a[4:9] == [2, 12, 128, 128, 64]
    assert a[9] == a[10] == a[11] == [128 * 2304, 64, 2304] and a[12] == [128 * 768, 64, 768]
    assert a[13] == pytest.approx(0.125)
    # any other number of keys fuses as well (the kernel walks them in blocks of 128) ...
    calls = _launches(donnx.ONNXModel("bert_s200", bert_encoder_layer_model(w, 2, 200, 12)))
    assert [f for f, _ in calls].count("mi355x_attention_f32") == 1 and len(calls) == 7
    a = [args for f, args in calls if f == "mi355x_attention_f32"][0]
    assert a[4:9] == [2, 12, 200, 200, 64]
    # ... another head size does not: the three nodes stay
    calls = _launches(donnx.ONNXModel("bert_d96", bert_encoder_layer_model(w, 2, 128, 8)))
    assert [f for f, _ in calls].count("mi355x_attention_f32") == 0 and len(calls) == 9


def test_shared_input_matmuls_with_other_readers_are_left_alone():
    # Y1 is also read by an Add: a column slice of a wide result cannot feed it without a copy
    rng = np.random.default_rng(1)
    w1, w2 = rng.normal(size=(8, 12)).astype(np.float32), rng.normal(size=(8, 12)).astype(np.float32)
    w3 = rng.normal(size=(12, 4)).astype(np.float32)
    nodes = [H.make_node("MatMul", ["x", "w1"], ["y1"]), H.make_node("MatMul", ["x", "w2"], ["y2"]),
             H.make_node("MatMul", ["y1", "w3"], ["z1"]), H.make_node("Add", ["y1", "y2"], ["s"])]
    g = H.make_graph(nodes, "g", [H.make_tensor_value_info("x", 1, [4, 8])],
                     [H.make_tensor_value_info("z1", 1, None), H.make_tensor_value_info("s", 1, None)],
                     initializer=[proto.numpy_helper.from_array(w1, "w1"), proto.numpy_helper.from_array(w2, "w2"),
                                  proto.numpy_helper.from_array(w3, "w3")])
    calls = _launches(donnx.ONNXModel("no_hfuse", H.make_model(g)))
    assert [f for f, _ in calls].count("mi355x_gemm_f32") == 3


def test_shared_input_matmuls_read_directly_by_matmuls_are_fused():
    rng = np.random.default_rng(2)
    w1, w2 = rng.normal(size=(8, 12)).astype(np.float32), rng.normal(size=(8, 4)).astype(np.float32)
    w3 = rng.normal(size=(12, 4)).astype(np.float32)
    nodes = [H.make_node("MatMul", ["x", "w1"], ["y1"]), H.make_node("MatMul", ["x", "w2"], ["y2"]),
             H.make_node("MatMul", ["y1", "w3"], ["z1"]), H.make_node("MatMul", ["w3", "y2"], ["z2"])]
    g = H.make_graph(nodes, "g", [H.make_tensor_value_info("x", 1, [4, 8])],
                     [H.make_tensor_value_info("z1", 1, None), H.make_tensor_value_info("z2", 1, None)],
                     initializer=[proto.numpy_helper.from_array(w1, "w1"), proto.numpy_helper.from_array(w2, "w2"),
                                  proto.numpy_helper.from_array(w3, "w3")])
    calls = _launches(donnx.ONNXModel("hfuse", H.make_model(g)))
    assert len(calls) == 3
    wide, z1, z2 = [a for _, a in calls]
    assert wide[5:10] == [1, 1, 4, 16, 8]
    assert z1[0].offset == 0 and z1[10] == [0, 0, 16, 1]      # y1 = columns 0..11 of the [4, 16] result
    assert z2[1].offset == 12 and z2[11] == [0, 0, 16, 1]     # y2 = columns 12..15, as the B operand


def test_decomposed_layernorm_and_gelu_are_recognised():
    # the opset-12 export form the reference executes node by node: 46 launches as written, 9 fused
    w = pure_ops.bert_layer_weights(np.random.default_rng(0), hidden=64, ffn=128)
    plain = [f for f, _ in _launches(donnx.ONNXModel("d0", bert_encoder_layer_model(w, 2, 16, 4, decomposed=True), fuse=False))]
    assert len(plain) == 46 and plain.count("mi355x_reduce_mean_f32") == 4
    fused = _launches(donnx.ONNXModel("d1", bert_encoder_layer_model(w, 2, 16, 4, decomposed=True)))
    names = [f for f, _ in fused]
    assert len(names) == 9 and names.count("mi355x_layernorm_f32") == 2 and names.count("mi355x_gemm_f32") == 6
    ln = [a for f, a in fused if f == "mi355x_layernorm_f32"][0]
    assert ln[4:6] == [32, 64] and ln[6] == pytest.approx(1e-12)
    assert sorted(a[15] for f, a in fused if f == "mi355x_gemm_f32") == [0, 0, 1, 5, 9, 9]   # Gelu folded into FFN1


def _chain_model(nodes, consts, shape=(4, 8)):
    g = H.make_graph(nodes, "g", [H.make_tensor_value_info("x", 1, list(shape))],
                     [H.make_tensor_value_info("y", 1, None)],
                     initializer=[proto.numpy_helper.from_array(np.array(v, dtype=np.float32), k) for k, v in consts.items()])
    return H.make_model(g)


def test_gelu_pattern_variants():
    consts = {"r2": 2.0 ** 0.5, "ir2": 0.5 ** 0.5, "one": 1.0, "half": 0.5}
    mk = H.make_node
    variants = {
        "div, (x * t) * 0.5": [mk("Div", ["x", "r2"], ["s"]), mk("Erf", ["s"], ["e"]), mk("Add", ["e", "one"], ["t"]),
                               mk("Mul", ["x", "t"], ["u"]), mk("Mul", ["u", "half"], ["y"])],
        "mul by 1/sqrt2, (t * 0.5) * x": [mk("Mul", ["ir2", "x"], ["s"]), mk("Erf", ["s"], ["e"]), mk("Add", ["one", "e"], ["t"]),
                                          mk("Mul", ["half", "t"], ["u"]), mk("Mul", ["u", "x"], ["y"])],
    }
    for label, nodes in variants.items():
        calls = _launches(donnx.ONNXModel("g", _chain_model(nodes, consts)))
        assert [(f, a[0]) for f, a in calls] == [("mi355x_eltwise_f32", 17)], label
    # a different constant is not Gelu: the five nodes are not replaced by the Gelu node (they still run as one
    # launch, as a program of five instructions)
    bad = dict(consts, r2=1.5)
    calls = _launches(donnx.ONNXModel("g", _chain_model(variants["div, (x * t) * 0.5"], bad)))
    assert [f for f, _ in calls] == ["mi355x_eltwise_program_f32"] and calls[0][1][8] == 5
    # erf(x / sqrt 2) with another reader of the intermediate is not Gelu either; both readers are elementwise,
    # so the value stays in a register of one five-instruction program
    nodes = variants["div, (x * t) * 0.5"][:-1] + [mk("Mul", ["u", "e"], ["y"])]
    calls = _launches(donnx.ONNXModel("g", _chain_model(nodes, consts)))
    assert [(f, a[8]) for f, a in calls] == [("mi355x_eltwise_program_f32", 5)]
    unfused = _launches(donnx.ONNXModel("g", _chain_model(nodes, consts), fuse=False))
    assert len(unfused) == 5


def _tanh_gelu_and_silu_nodes():
    """x -> tanh-approximated Gelu (eight elementwise nodes) -> SiLU (x * sigmoid(x)) -> Softplus."""
    mk = H.make_node
    consts = {"c": 0.044715, "k": (2.0 / np.pi) ** 0.5, "one": 1.0, "half": 0.5, "three": 3.0}
    nodes = [mk("Pow", ["x", "three"], ["x3"]), mk("Mul", ["x3", "c"], ["cx3"]), mk("Add", ["x", "cx3"], ["inner"]),
             mk("Mul", ["inner", "k"], ["scaled"]), mk("Tanh", ["scaled"], ["t"]), mk("Add", ["t", "one"], ["t1"]),
             mk("Mul", ["x", "t1"], ["xt"]), mk("Mul", ["xt", "half"], ["gelu"]),
             mk("Sigmoid", ["gelu"], ["sg"]), mk("Mul", ["gelu", "sg"], ["silu"]), mk("Softplus", ["silu"], ["y"])]
    return nodes, consts


def test_tanh_sigmoid_softplus_chains_become_one_program():
    # the unary maps of pure_implementations.py:275-298, 696-712 join elementwise groups like Relu / Erf / Sqrt do
    nodes, consts = _tanh_gelu_and_silu_nodes()
    calls = _launches(donnx.ONNXModel("g", _chain_model(nodes, consts)))
    assert [f for f, _ in calls] == ["mi355x_eltwise_program_f32"] and calls[0][1][8] == 11
    assert calls[0][1][1] == 1 and calls[0][1][3] == 0           # one tensor read, no vectors
    unfused = _launches(donnx.ONNXModel("g", _chain_model(nodes, consts), fuse=False))
    assert [f for f, _ in unfused] == ["mi355x_eltwise_f32"] * 11
    assert sorted(a[0] for _, a in unfused) == sorted([4, 2, 0, 2, 22, 0, 2, 2, 23, 2, 24])


def test_elementwise_groups_respect_the_kernel_limits_and_outside_readers():
    mk = H.make_node
    # 20 dependent nodes: more than one program holds (16 instructions) -> two programs, 20 instructions in all
    nodes = [mk("Tanh" if i % 2 else "Abs", ["x" if i == 0 else f"v{i - 1}"], [f"v{i}" if i < 19 else "y"]) for i in range(20)]
    calls = _launches(donnx.ONNXModel("g", _chain_model(nodes, {})))
    assert [f for f, _ in calls] == ["mi355x_eltwise_program_f32"] * 2 and sum(a[8] for _, a in calls) == 20
    assert max(a[8] for _, a in calls) <= 16
    # nine values alive at once do not fit eight registers: the group shrinks until it does
    nodes = [mk("Tanh" if i % 2 else "Abs", ["x"], [f"b{i}"]) for i in range(9)]
    nodes += [mk("Sigmoid", [f"b{i}"], [f"c{i}"]) for i in range(9)]
    acc = "c0"
    for i in range(1, 9):
        nodes.append(mk("Mul", [acc, f"c{i}"], [f"m{i}" if i < 8 else "y"]))
        acc = f"m{i}"
    model = donnx.ONNXModel("g", _chain_model(nodes, {}))
    calls = _launches(model)
    assert sum(a[8] if f == "mi355x_eltwise_program_f32" else 1 for f, a in calls) == 26 and len(calls) <= 4
    for f, a in calls:
        assert f == "mi355x_eltwise_f32" or (a[8] <= 16 and max((w >> 8) & 255 for w in a[7].values) < 8)
    # an intermediate that something outside the group reads (here: a MatMul) is materialised, not absorbed
    nodes = [mk("Tanh", ["x"], ["t"]), mk("Sigmoid", ["t"], ["s"]), mk("Mul", ["t", "s"], ["p"]),
             mk("MatMul", ["t", "w"], ["q"]), mk("Add", ["p", "q"], ["y"])]
    g = _chain_model(nodes, {"w": np.eye(8)})
    calls = _launches(donnx.ONNXModel("g", g))
    assert sorted(f for f, _ in calls) == ["mi355x_eltwise_f32", "mi355x_eltwise_program_f32", "mi355x_gemm_f32"]


def test_layernorm_pattern_needs_the_exact_chain():
    mk = H.make_node
    consts = {"two": 2.0, "three": 3.0, "eps": 1e-5, "g": np.ones(8), "b": np.zeros(8)}

    def chain(exponent="two", axes=(-1, )):
        return [mk("ReduceMean", ["x"], ["m"], axes=list(axes), keepdims=1), mk("Sub", ["x", "m"], ["c"]),
                mk("Pow", ["c", exponent], ["p"]), mk("ReduceMean", ["p"], ["v"], axes=list(axes), keepdims=1),
                mk("Add", ["v", "eps"], ["ve"]), mk("Sqrt", ["ve"], ["s"]), mk("Div", ["c", "s"], ["n"]),
                mk("Mul", ["n", "g"], ["sc"]), mk("Add", ["sc", "b"], ["y"])]

    calls = _launches(donnx.ONNXModel("ln", _chain_model(chain(), consts)))
    assert [f for f, _ in calls] == ["mi355x_layernorm_f32"] and calls[0][1][6] == pytest.approx(1e-5)
    # not the LayerNorm chain (cube instead of square; statistics over axis 0): no LayerNormalization node. What
    # can run as an elementwise program does: Add(eps)+Sqrt, and the tail Mul(gamma)+Add(beta) -- with the Div in
    # front of it when its divisor is a vector along the last axis (axis-0 statistics) rather than one value
    # per row, a broadcast the program kernel does not do
    cube = [f for f, _ in _launches(donnx.ONNXModel("ln3", _chain_model(chain(exponent="three"), consts)))]
    assert "mi355x_layernorm_f32" not in cube and len(cube) == 7 and cube.count("mi355x_eltwise_program_f32") == 2
    axis0 = _launches(donnx.ONNXModel("ln0", _chain_model(chain(axes=(0, )), dict(consts, g=np.ones(8)))))
    assert "mi355x_layernorm_f32" not in [f for f, _ in axis0] and len(axis0) == 6
    assert sorted(a[8] for f, a in axis0 if f == "mi355x_eltwise_program_f32") == [2, 3]


def test_rebase_and_reshape_strides():
    # [B, H, S, D] view of a contiguous [B*S, 768] array, moved into a [B*S, 2304] array
    assert _rebase_strides([8, 12, 128, 64], [98304, 64, 768, 1], 768, 2304) == [294912, 64, 2304, 1]
    # a dimension that neither steps whole rows nor stays inside one
    assert _rebase_strides([4, 100], [100, 1], 64, 128) is None
    # numpy's no-copy reshape rule
    assert _reshape_strides([8, 128, 768], [98304, 768, 1], [8, 128, 12, 64]) == [98304, 768, 64, 1]
    assert _reshape_strides([8, 12, 128, 64], [98304, 64, 768, 1], [8, 12, 8192]) is None
    a = np.arange(24).reshape(2, 3, 4)
    v = a.transpose(1, 0, 2)
    assert _reshape_strides(list(v.shape), [s // 8 for s in v.strides], [3, 8]) is None  # numpy would copy
    assert _reshape_strides([2, 3, 4], [12, 4, 1], [6, 4]) == [4, 1]


def test_scalar_scale_on_an_operand_becomes_alpha():
    T = proto.TensorProto
    def model(op, const_first):
        ins = ["c", "q"] if const_first else ["q", "c"]
        nodes = [H.make_node(op, ins, ["qs"]), H.make_node("Transpose", ["k"], ["kt"], perm=[0, 2, 1]),
                 H.make_node("MatMul", ["qs", "kt"], ["y"])]
        g = H.make_graph(nodes, "g", [H.make_tensor_value_info("q", T.FLOAT, [3, 8, 16]),
                                      H.make_tensor_value_info("k", T.FLOAT, [3, 12, 16])],
                         [H.make_tensor_value_info("y", T.FLOAT, [3, 8, 12])],
                         initializer=[proto.numpy_helper.from_array(np.array(0.25, np.float32), name="c")])
        return donnx.ONNXModel("scaled_" + op + str(const_first), H.make_model(g, opset_imports=[H.make_opsetid("", 12)]))

    for op, const_first, alpha in (("Mul", False, 0.25), ("Mul", True, 0.25), ("Div", False, 4.0)):
        calls = _launches(model(op, const_first))
        assert [f for f, _ in calls] == ["mi355x_gemm_f32"], (op, const_first)
        assert alpha in calls[0][1]
    # a constant numerator is not a scale of the operand: c / q stays an elementwise launch
    assert [f for f, _ in _launches(model("Div", True))] == ["mi355x_eltwise_f32", "mi355x_gemm_f32"]


def test_gemm_with_a_full_addend_does_not_take_an_activation():
    # the epilogue order is bias, activation, residual; Gemm's C of shape [M, N] travels as the residual, so
    # Relu(A B + C) must stay two launches, while a row bias C of shape [N] folds
    T = proto.TensorProto
    def model(c_shape):
        nodes = [H.make_node("Gemm", ["a", "b", "c"], ["g"]), H.make_node("Relu", ["g"], ["y"])]
        g = H.make_graph(nodes, "g", [H.make_tensor_value_info("a", T.FLOAT, [6, 8]), H.make_tensor_value_info("b", T.FLOAT, [8, 12]),
                                      H.make_tensor_value_info("c", T.FLOAT, c_shape)],
                         [H.make_tensor_value_info("y", T.FLOAT, [6, 12])])
        return donnx.ONNXModel("gemm_relu_" + str(len(c_shape)), H.make_model(g, opset_imports=[H.make_opsetid("", 12)]))
    assert [f for f, _ in _launches(model([12]))] == ["mi355x_gemm_f32"]
    assert [f for f, _ in _launches(model([1, 12]))] == ["mi355x_gemm_f32"]
    assert [f for f, _ in _launches(model([6, 12]))] == ["mi355x_gemm_f32", "mi355x_eltwise_f32"]


def _pad_conv_model(pads, value=0.0, mode="constant", conv_pads=None, second_reader=False):
    T = proto.TensorProto
    rng = np.random.default_rng(5)
    inits = [proto.numpy_helper.from_array(np.array(pads, np.int64), name="pads"),
             proto.numpy_helper.from_array(np.array(value, np.float32), name="zero"),
             proto.numpy_helper.from_array(rng.normal(size=(4, 3, 3, 3)).astype(np.float32), name="w")]
    out_hw = [8 + pads[2] + pads[6] + (conv_pads[0] + conv_pads[2] if conv_pads else 0) - 2,
              8 + pads[3] + pads[7] + (conv_pads[1] + conv_pads[3] if conv_pads else 0) - 2]
    attrs = {"pads": conv_pads} if conv_pads else {}
    nodes = [H.make_node("Pad", ["x", "pads", "zero"], ["xp"], mode=mode), H.make_node("Conv", ["xp", "w"], ["y"], **attrs)]
    outs = [H.make_tensor_value_info("y", T.FLOAT, [2, 4] + out_hw)]
    if second_reader:
        nodes.append(H.make_node("Relu", ["xp"], ["r"]))
        outs.append(H.make_tensor_value_info("r", T.FLOAT, None))
    g = H.make_graph(nodes, "g", [H.make_tensor_value_info("x", T.FLOAT, [2, 3, 8, 8])], outs, initializer=inits)
    return H.make_model(g, opset_imports=[H.make_opsetid("", 12)])


def test_pad_conv_fusion():
    # the reference's PadConvFusion: a constant zero pad of H and W folds into the convolution's pads
    calls = _launches(donnx.ONNXModel("pad_conv", _pad_conv_model([0, 0, 1, 2, 0, 0, 3, 0])))
    assert [f for f, _ in calls] == ["mi355x_conv2d_f32"]
    assert [1, 2, 3, 0] in calls[0][1]                       # pads {top, left, bottom, right}
    calls = _launches(donnx.ONNXModel("pad_conv2", _pad_conv_model([0, 0, 1, 1, 0, 0, 1, 1], conv_pads=[1, 0, 0, 2])))
    assert [2, 1, 1, 3] in calls[0][1]                       # added to the pads the Conv already had
    # not foldable: a non-zero value, another mode, padding along channels, a second reader of the padded tensor;
    # a Pad that stays has no kernel here and is refused when it is expanded
    from dace_onnx_amd.onnx.nodes.onnx_op import ExpansionRefused
    for kwargs in (dict(pads=[0, 0, 1, 1, 0, 0, 1, 1], value=1.0), dict(pads=[0, 0, 1, 1, 0, 0, 1, 1], mode="reflect"),
                   dict(pads=[0, 1, 1, 1, 0, 0, 1, 1]), dict(pads=[0, 0, 1, 1, 0, 0, 1, 1], second_reader=True)):
        model = donnx.ONNXModel("pad_kept", _pad_conv_model(**kwargs))
        with pytest.raises(ExpansionRefused, match="Pad"):
            model.expand()


def _conv_bn_model(conv_bias=True, second_reader=False, variable_scale=False, relu=True):
    T = proto.TensorProto
    rng = np.random.default_rng(7)
    w = rng.normal(size=(4, 3, 3, 3)).astype(np.float32)
    params = {"scale": rng.normal(size=4), "beta": rng.normal(size=4), "mean": rng.normal(size=4), "var": rng.uniform(0.5, 2.0, size=4),
              "cb": rng.normal(size=4)}
    inits = [proto.numpy_helper.from_array(w, name="w")] + \
        [proto.numpy_helper.from_array(v.astype(np.float32), name=k) for k, v in params.items() if not (variable_scale and k == "scale")]
    nodes = [H.make_node("Conv", ["x", "w"] + (["cb"] if conv_bias else []), ["c"], pads=[1, 1, 1, 1]),
             H.make_node("BatchNormalization", ["c", "scale", "beta", "mean", "var"], ["b"], epsilon=1e-3)]
    ins = [H.make_tensor_value_info("x", T.FLOAT, [2, 3, 8, 8])]
    if variable_scale:
        ins.append(H.make_tensor_value_info("scale", T.FLOAT, [4]))
    outs = []
    if relu:
        nodes.append(H.make_node("Relu", ["b"], ["y"]))
    if second_reader:
        nodes.append(H.make_node("Relu", ["c"], ["r"]))
        outs.append(H.make_tensor_value_info("r", T.FLOAT, None))
    outs.insert(0, H.make_tensor_value_info("y" if relu else "b", T.FLOAT, [2, 4, 8, 8]))
    g = H.make_graph(nodes, "g", ins, outs, initializer=inits)
    return H.make_model(g, opset_imports=[H.make_opsetid("", 12)]), w, {k: v.astype(np.float32) for k, v in params.items()}


def test_batchnorm_folds_into_the_convolution():
    # Conv -> BatchNormalization (inference, constant parameters) -> Relu is one convolution launch with new weights
    for conv_bias in (True, False):
        m, w, p = _conv_bn_model(conv_bias=conv_bias)
        model = donnx.ONNXModel(f"conv_bn_{conv_bias}", m)
        calls = _launches(model)
        assert [f for f, _ in calls] == ["mi355x_conv2d_f32"]
        a = p["scale"].astype(np.float64) / np.sqrt(p["var"].astype(np.float64) + 1e-3)
        folded_w = [v for k, v in model.weights.items() if "_bnfold_" in k and "bias" not in k][0].cpu().numpy()
        folded_b = [v for k, v in model.weights.items() if "_bnfold_bias_" in k][0].cpu().numpy()
        assert np.allclose(folded_w, w * a.reshape(-1, 1, 1, 1), rtol=1e-6)
        assert np.allclose(folded_b, ((p["cb"] if conv_bias else 0.0) - p["mean"]) * a + p["beta"], rtol=1e-5, atol=1e-6)
        assert np.array_equal(model.weights["w"].cpu().numpy(), w)          # the original stays as it was
    # not folded: the convolution's result has another reader, or a parameter is a graph input
    for kwargs in (dict(second_reader=True), dict(variable_scale=True)):
        calls = _launches(donnx.ONNXModel("conv_bn_kept", _conv_bn_model(**kwargs)[0]))
        assert "mi355x_batchnorm_f32" in [f for f, _ in calls]
    unfused = _launches(donnx.ONNXModel("conv_bn_plain", _conv_bn_model()[0], fuse=False))
    assert [f for f, _ in unfused] == ["mi355x_conv2d_f32", "mi355x_batchnorm_f32", "mi355x_eltwise_f32"]


def _tasklet_fusion_graphs():
    """The three programs of the reference's tests/transformation/test_tasklet_fusion.py, as ONNX graphs:
    (A + 1) * 2, (A + 1) + (A * 3), (A + 1) + (B * 3)."""
    mk, T = H.make_node, proto.TensorProto
    consts = [proto.numpy_helper.from_array(np.array(v, np.float32), k) for k, v in (("one", 1.0), ("two", 2.0), ("three", 3.0))]
    graphs = {
        "basic": ([mk("Add", ["A", "one"], ["b"]), mk("Mul", ["b", "two"], ["y"])], ["A"], lambda A, B: (A + 1) * 2),
        "same_name": ([mk("Add", ["A", "one"], ["b"]), mk("Mul", ["A", "three"], ["c"]), mk("Add", ["b", "c"], ["y"])], ["A"],
                      lambda A, B: A + 1 + A * 3),
        "same_name_diff_memlet": ([mk("Add", ["A", "one"], ["d"]), mk("Mul", ["B", "three"], ["c"]), mk("Add", ["d", "c"], ["y"])],
                                  ["A", "B"], lambda A, B: A + 1 + B * 3),
    }
    out = {}
    for name, (nodes, inputs, fn) in graphs.items():
        g = H.make_graph(nodes, name, [H.make_tensor_value_info(i, T.FLOAT, [5, 5]) for i in inputs],
                         [H.make_tensor_value_info("y", T.FLOAT, [5, 5])], initializer=consts)
        out[name] = (H.make_model(g, opset_imports=[H.make_opsetid("", 12)]), inputs, fn)
    return out


def test_tasklet_fusion_programs_become_one_launch():
    for name, (m, inputs, _) in _tasklet_fusion_graphs().items():
        calls = _launches(donnx.ONNXModel("tf_" + name, m))
        assert [f for f, _ in calls] == ["mi355x_eltwise_program_f32"], name
        assert calls[0][1][1] == len(inputs) and calls[0][1][8] == len(m.graph.node)     # tensors read, instructions


@pytest.mark.parametrize("opset, expected", [(12, (2, 3, 8)), (13, (6, 8, 1)), (17, (6, 8, 1))])
@pytest.mark.parametrize("op", ["Softmax", "LogSoftmax"])
def test_softmax_without_axis_attribute_takes_the_default_of_the_models_opset(op, opset, expected):
    """The operator's default axis is 1 up to opset 12 and the last axis from opset 13 on; the reference only
    ever sees opset 12 (daceml/pytorch/module.py:248), this importer also accepts 17 and 20."""
    g = H.make_graph([H.make_node(op, ["x"], ["y"])], "g", [H.make_tensor_value_info("x", 1, [2, 3, 8])],
                     [H.make_tensor_value_info("y", 1, [2, 3, 8])])
    calls = _launches(donnx.ONNXModel(f"{op}_{opset}", H.make_model(g, opset_imports=[H.make_opsetid("", opset)])))
    assert len(calls) == 1 and calls[0][0] == ("mi355x_softmax_f32" if op == "Softmax" else "mi355x_log_softmax_f32")
    assert tuple(calls[0][1][2:5]) == expected   # outer, axis_len, inner
    # an explicit attribute wins in every opset
    g = H.make_graph([H.make_node(op, ["x"], ["y"], axis=0)], "g", [H.make_tensor_value_info("x", 1, [2, 3, 8])],
                     [H.make_tensor_value_info("y", 1, [2, 3, 8])])
    calls = _launches(donnx.ONNXModel(f"{op}_{opset}_a0", H.make_model(g, opset_imports=[H.make_opsetid("", opset)])))
    assert tuple(calls[0][1][2:5]) == (1, 2, 24)

"""Builders of the benchmark ONNX graphs (as ``ModelProto`` objects).

``bert_encoder_layer_model`` is the BERT-base encoder layer the reference tests
through ``DaceModule(BertLayer(BertConfig()))`` (tests/pytorch/test_bert_encoder.py:10-34),
written directly as the ONNX graph of MatMul / Add / Reshape / Transpose / Div /
Softmax / LayerNormalization / Gelu nodes, with weights stored ``[in, out]`` as
MatMul consumes them.
"""
import math

import numpy as np

from ..onnx.proto import helper, numpy_helper, TensorProto


def bert_encoder_layer_model(w, batch, seq, heads, eps=1e-12, name="bert_encoder_layer", decomposed=False):
    """:param w: dict with wq wk wv wo [H,H], w1 [H,F], w2 [F,H], biases bq bk bv bo b1 b2,
                 ln1_g ln1_b ln2_g ln2_b (see ``oracle.pure_ops.bert_layer_weights``).
       :param decomposed: write LayerNorm and Gelu the way an opset-12 export does (the form the
                 reference executes): ReduceMean, Sub, Pow, ReduceMean, Add, Sqrt, Div, Mul, Add and
                 Div, Erf, Add, Mul, Mul."""
    hidden = w["wq"].shape[0]
    d = hidden // heads
    f32 = TensorProto.FLOAT
    inits = [numpy_helper.from_array(np.asarray(v, dtype=np.float32), k) for k, v in w.items()]
    inits += [
        numpy_helper.from_array(np.array([batch, seq, heads, d], dtype=np.int64), "split_shape"),
        numpy_helper.from_array(np.array([batch, seq, hidden], dtype=np.int64), "merge_shape"),
        numpy_helper.from_array(np.array(math.sqrt(d), dtype=np.float32), "sqrt_d"),
    ]
    nodes = []

    def n(op, ins, out, **attrs):
        nodes.append(helper.make_node(op, ins, [out], name=f"{op}_{len(nodes)}", **attrs))
        return out

    def proj(x, wn, bn, tag):
        return n("Add", [n("MatMul", [x, wn], f"{tag}_mm"), bn], f"{tag}_lin")

    def split_heads(x, tag):
        r = n("Reshape", [x, "split_shape"], f"{tag}_4d")
        return n("Transpose", [r], f"{tag}_heads", perm=[0, 2, 1, 3])

    q = split_heads(proj("x", "wq", "bq", "q"), "q")
    k = split_heads(proj("x", "wk", "bk", "k"), "k")
    v = split_heads(proj("x", "wv", "bv", "v"), "v")
    kt = n("Transpose", [k], "k_t", perm=[0, 1, 3, 2])
    scores = n("Div", [n("MatMul", [q, kt], "scores_raw"), "sqrt_d"], "scores")
    probs = n("Softmax", [scores], "probs", axis=3)
    ctx = n("MatMul", [probs, v], "ctx_heads")
    ctx = n("Reshape", [n("Transpose", [ctx], "ctx_t", perm=[0, 2, 1, 3]), "merge_shape"], "ctx")
    def layer_norm(x, g, b, out, tag):
        if not decomposed:
            return n("LayerNormalization", [x, g, b], out, axis=-1, epsilon=eps)
        mean = n("ReduceMean", [x], f"{tag}_mean", axes=[-1], keepdims=1)
        centred = n("Sub", [x, mean], f"{tag}_centred")
        var = n("ReduceMean", [n("Pow", [centred, "two"], f"{tag}_sq")], f"{tag}_var", axes=[-1], keepdims=1)
        std = n("Sqrt", [n("Add", [var, "ln_eps"], f"{tag}_var_eps")], f"{tag}_std")
        normed = n("Div", [centred, std], f"{tag}_normed")
        return n("Add", [n("Mul", [normed, g], f"{tag}_scaled"), b], out)

    def gelu(x, out):
        if not decomposed:
            return n("Gelu", [x], out)
        t = n("Add", [n("Erf", [n("Div", [x, "sqrt_2"], f"{out}_scaled")], f"{out}_erf"), "one"], f"{out}_erf1")
        return n("Mul", [n("Mul", [x, t], f"{out}_xerf"), "half"], out)

    if decomposed:
        inits += [numpy_helper.from_array(np.array(v, dtype=np.float32), k) for k, v in
                  (("two", 2.0), ("ln_eps", eps), ("sqrt_2", math.sqrt(2.0)), ("one", 1.0), ("half", 0.5))]
    attn = proj(ctx, "wo", "bo", "attn")
    h1 = layer_norm(n("Add", [attn, "x"], "attn_res"), "ln1_g", "ln1_b", "h1", "ln1")
    inter = gelu(proj(h1, "w1", "b1", "ffn1"), "inter")
    out = proj(inter, "w2", "b2", "ffn2")
    layer_norm(n("Add", [out, h1], "ffn_res"), "ln2_g", "ln2_b", "y", "ln2")

    graph = helper.make_graph(nodes, name,
                              [helper.make_tensor_value_info("x", f32, [batch, seq, hidden])],
                              [helper.make_tensor_value_info("y", f32, [batch, seq, hidden])],
                              initializer=inits)
    return helper.make_model(graph, opset_imports=[helper.make_opsetid("", 12 if decomposed else 17)])


def conv_relu_model(W, bias, x_shape, pads=(1, 1, 1, 1), strides=(1, 1), name="conv_relu"):
    """ResNet-style Conv + Relu (benchmark config 4)."""
    f32 = TensorProto.FLOAT
    inits = [numpy_helper.from_array(np.asarray(W, dtype=np.float32), "W")]
    ins = ["X", "W"]
    if bias is not None:
        inits.append(numpy_helper.from_array(np.asarray(bias, dtype=np.float32), "B"))
        ins.append("B")
    nodes = [helper.make_node("Conv", ins, ["conv_out"], name="conv", pads=list(pads), strides=list(strides),
                              kernel_shape=list(W.shape[2:])),
             helper.make_node("Relu", ["conv_out"], ["Y"], name="relu")]
    graph = helper.make_graph(nodes, name, [helper.make_tensor_value_info("X", f32, list(x_shape))],
                              [helper.make_tensor_value_info("Y", f32, None)], initializer=inits)
    return helper.make_model(graph)

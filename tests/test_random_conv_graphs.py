"""Random convolution-network graphs: the fused graph, the node-by-node graph and the oracle's evaluation of
the same node list must agree.

What the fusion pass does to such graphs -- BatchNormalization folded into the weights of the Conv before it,
Relu / a same-shape Add / the Relu after it folded into the Conv's epilogue, Pad into its pads, leftover
elementwise nodes grouped into programs -- must never change the value, whatever else reads the tensors in
between. Each seeded graph is a random walk over Conv (with or without bias, 1 x 1 or 3 x 3, strides),
BatchNormalization, Relu / Sigmoid / Tanh, residual Adds with earlier values of the same shape (either operand
order), MaxPool, values with several readers, and ends in GlobalAveragePool, Flatten, Gemm, LogSoftmax. Without a
GPU the graphs are imported, fused and expanded (structure only); with one, all three results are compared."""
import numpy as np
import pytest

from dace_onnx_amd import sdfg as dace
import dace_onnx_amd.onnx as donnx
from dace_onnx_amd.onnx import proto
from oracle import pure_ops as O
from conftest import rel_err, FP32_REL_TOL

H, T = proto.helper, proto.TensorProto


def random_conv_graph(seed):
    rng = np.random.default_rng(seed)
    nodes, inits, shapes, count = [], [], {}, [0]

    def name(hint):
        count[0] += 1
        return f"{hint}_{count[0]}"

    def const(value, hint):
        n = name(hint)
        inits.append(proto.numpy_helper.from_array(np.asarray(value, dtype=np.float32), name=n))
        return n

    def node(op, ins, shape, **attrs):
        out = name(op.lower())
        nodes.append(H.make_node(op, list(ins), [out], name=name("n"), **attrs))
        shapes[out] = tuple(shape)
        return out

    batch, channels, size = int(rng.choice([1, 2, 3])), int(rng.choice([3, 8, 16])), int(rng.choice([8, 12, 17]))
    x_shape = (batch, channels, size, size)
    shapes["x"] = x_shape
    cur, pool = "x", ["x"]
    for _ in range(int(rng.integers(3, 9))):
        n, c, h, w = shapes[cur]
        kind = rng.choice(["conv", "conv", "conv", "bn", "act", "residual", "maxpool", "reuse"])
        if kind == "conv":
            k = int(rng.choice([1, 3]))
            stride = int(rng.choice([1, 1, 2])) if min(h, w) >= 6 else 1
            oc = int(rng.choice([4, 8, 16, c]))
            pad = k // 2
            ins = [cur, const(rng.normal(0, 1.0 / np.sqrt(c * k * k), size=(oc, c, k, k)), "w")]
            if rng.random() < 0.6:
                ins.append(const(rng.normal(0, 0.1, size=oc), "b"))
            cur = node("Conv", ins, (n, oc, (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1),
                       kernel_shape=[k, k], pads=[pad] * 4, strides=[stride, stride])
        elif kind == "bn":
            params = [const(rng.normal(1, 0.2, size=c), "scale"), const(rng.normal(0, 0.2, size=c), "beta"),
                      const(rng.normal(0, 0.3, size=c), "mean"), const(rng.uniform(0.5, 2.0, size=c), "var")]
            cur = node("BatchNormalization", [cur] + params, shapes[cur], epsilon=float(rng.choice([1e-5, 1e-3])))
        elif kind == "act":
            cur = node(str(rng.choice(["Relu", "Relu", "Sigmoid", "Tanh"])), [cur], shapes[cur])
        elif kind == "residual":
            same = [p for p in pool if shapes[p] == shapes[cur] and p != cur]
            if same:
                other = str(rng.choice(same))
                cur = node("Add", [cur, other] if rng.random() < 0.5 else [other, cur], shapes[cur])
        elif kind == "maxpool" and min(h, w) >= 4:
            k, stride = int(rng.choice([2, 3])), int(rng.choice([1, 2]))
            pad = int(rng.integers(0, k // 2 + 1))
            cur = node("MaxPool", [cur], (n, c, (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1),
                       kernel_shape=[k, k], strides=[stride, stride], pads=[pad] * 4)
        elif kind == "reuse":
            a = node("Relu", [cur], shapes[cur])
            b = node("Mul", [cur, const(np.float32(0.5), "half")], shapes[cur])
            cur = node("Add", [a, b], shapes[cur])
        pool.append(cur)
    n, c, h, w = shapes[cur]
    g = node("GlobalAveragePool", [cur], (n, c, 1, 1))
    f = node("Flatten", [g], (n, c), axis=1)
    logits = node("Gemm", [f, const(rng.normal(0, 0.3, size=(10, c)), "wf"), const(rng.normal(0, 0.1, size=10), "bf")], (n, 10), transB=1)
    out = node("LogSoftmax", [logits], (n, 10), axis=1)
    graph = H.make_graph(nodes, f"random_conv_{seed}", [H.make_tensor_value_info("x", T.FLOAT, list(x_shape))],
                         [H.make_tensor_value_info(out, T.FLOAT, [n, 10])], initializer=inits)
    return H.make_model(graph, opset_imports=[H.make_opsetid("", 12)]), x_shape


def evaluate_with_oracle(model, x):
    env = {t.name: np.asarray(t.array).reshape(t.dims) for t in model.graph.initializer}
    env["x"] = x
    for n in model.graph.node:
        a = {at.name: at.value for at in n.attribute}
        i = [env[k] for k in n.input]
        op = n.op_type
        if op == "Conv":
            y = O.conv2d(i[0], i[1], i[2] if len(i) > 2 else None, strides=tuple(a["strides"]), pads=tuple(a["pads"]))
        elif op == "BatchNormalization":
            y = O.batch_normalization(i[0], i[1], i[2], i[3], i[4], float(a["epsilon"]))
        elif op in ("Relu", "Sigmoid", "Tanh"):
            y = getattr(O, op.lower())(i[0])
        elif op in ("Add", "Mul"):
            y = getattr(O, op.lower())(i[0], i[1])
        elif op == "MaxPool":
            y = O.maxpool2d(i[0], tuple(a["kernel_shape"]), tuple(a["strides"]), tuple(a["pads"]))
        elif op == "GlobalAveragePool":
            y = O.global_average_pool(i[0])
        elif op == "Flatten":
            y = i[0].reshape(i[0].shape[0], -1)
        elif op == "Gemm":
            y = O.gemm(i[0], i[1], i[2], transB=int(a.get("transB", 0)))
        elif op == "LogSoftmax":
            y = O.log_softmax(i[0], axis=int(a["axis"]))
        else:
            raise AssertionError(op)
        env[n.output[0]] = y
    return env[model.graph.output[0].name]


SEEDS = list(range(40))


@pytest.mark.parametrize("seed", SEEDS)
def test_random_conv_graph_fuses_and_expands(seed):
    model, _ = random_conv_graph(seed)
    fused = donnx.ONNXModel(f"rc_fused_{seed}", model)
    plain = donnx.ONNXModel(f"rc_plain_{seed}", model, fuse=False)
    n_fused = sum(isinstance(n, dace.KernelCall) for n, _ in fused.expand().all_nodes_recursive())
    n_plain = sum(isinstance(n, dace.KernelCall) for n, _ in plain.expand().all_nodes_recursive())
    assert 1 <= n_fused <= n_plain
    for m in (fused, plain):
        assert not any(isinstance(n, dace.LibraryNode) for n, _ in m.sdfg.all_nodes_recursive())


@pytest.mark.gpu
@pytest.mark.parametrize("seed", SEEDS)
def test_random_conv_graph_values(seed):
    model, x_shape = random_conv_graph(seed)
    x = np.random.default_rng(2000 + seed).normal(size=x_shape).astype(np.float32)
    expected = evaluate_with_oracle(model, x)
    print(f"random conv graph seed {seed}: {[n.op_type for n in model.graph.node]}", flush=True)
    fused = donnx.ONNXModel(f"rc_fused_{seed}", model)(x)
    plain = donnx.ONNXModel(f"rc_plain_{seed}", model, fuse=False)(x)
    assert rel_err(expected, plain) < FP32_REL_TOL
    assert rel_err(expected, fused) < FP32_REL_TOL

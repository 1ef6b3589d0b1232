"""Random ONNX graphs over the hot-path operators: the fused graph, the node-by-node graph and the oracle's
evaluation of the same node list must agree.

The fusion pass rewrites chains (bias / scale / activation / residual into GEMM epilogues, Reshape and
Transpose into operand strides, shared-input MatMuls into one, attention into one node); what it must
never do is change the value. Each seeded graph is a random walk over MatMul (constant weight, optional
bias as either Add operand), Gemm, scalar Mul / Div before or after a product, Relu / Gelu / Tanh / Sigmoid /
Softplus / Abs / Neg, residual Adds
with earlier values, LayerNormalization, Softmax, head split / merge (Reshape + Transpose) and
activation-by-activation MatMuls, with values that have several readers now and then. Without a GPU the
graphs are imported, fused and expanded (structure only); with one, all three results are compared."""
import numpy as np
import pytest

from dace_onnx_amd import sdfg as dace
import dace_onnx_amd.onnx as donnx
from dace_onnx_amd.onnx import proto
from oracle import pure_ops as O
from conftest import rel_err, FP32_REL_TOL

H, T = proto.helper, proto.TensorProto


class _Builder:
    def __init__(self, rng):
        self.rng, self.nodes, self.inits, self.count = rng, [], [], 0
        self.shapes = {}

    def name(self, hint):
        self.count += 1
        return f"{hint}_{self.count}"

    def const(self, value, hint="c"):
        n = self.name(hint)
        value = np.asarray(value, dtype=np.float32) if not isinstance(value, np.ndarray) or value.dtype != np.int64 else value
        self.inits.append(proto.numpy_helper.from_array(value, name=n))
        self.shapes[n] = tuple(value.shape)
        return n

    def node(self, op, ins, shape, **attrs):
        out = self.name(op.lower())
        self.nodes.append(H.make_node(op, list(ins), [out], name=self.name("n"), **attrs))
        self.shapes[out] = tuple(shape)
        return out


def random_graph(seed):
    """(model, input shape): a chain of 4-10 steps on a [B, S, Hd] activation."""
    rng = np.random.default_rng(seed)
    g = _Builder(rng)
    batch, seq = int(rng.choice([1, 2, 3])), int(rng.choice([4, 16, 20, 128]))
    hidden = int(rng.choice([32, 64, 128]))
    x_shape = (batch, seq, hidden)
    g.shapes["x"] = x_shape
    cur, pool = "x", ["x"]

    def weight(k, n):
        return g.const(rng.normal(0, 1.0 / np.sqrt(k), size=(k, n)).astype(np.float32), "w")

    def linear(src, n_out):
        shape = g.shapes[src]
        y = g.node("MatMul", [src, weight(shape[-1], n_out)], shape[:-1] + (n_out, ))
        if rng.random() < 0.7:
            b = g.const(rng.normal(0, 0.1, size=n_out).astype(np.float32), "b")
            y = g.node("Add", [y, b] if rng.random() < 0.5 else [b, y], g.shapes[y])
        return y

    for _ in range(int(rng.integers(4, 11))):
        shape = g.shapes[cur]
        kind = rng.choice(["linear", "linear", "act", "scale", "residual", "ln", "softmax", "attention", "gemm", "reuse"])
        if kind == "linear":
            cur = linear(cur, int(rng.choice([32, 64, 96, 128])))
        elif kind == "act":
            cur = g.node(str(rng.choice(["Relu", "Gelu", "Tanh", "Sigmoid", "Softplus", "Abs", "Neg"])), [cur], shape)
        elif kind == "scale":
            c = g.const(np.float32(rng.choice([0.5, 2.0, 0.125, -1.5])), "s")
            op = str(rng.choice(["Mul", "Div"]))
            cur = g.node(op, [cur, c] if op == "Div" or rng.random() < 0.5 else [c, cur], shape)
        elif kind == "residual":
            same = [p for p in pool if g.shapes[p] == shape and p != cur]
            if same:
                other = str(rng.choice(same))
                cur = g.node("Add", [cur, other] if rng.random() < 0.5 else [other, cur], shape)
        elif kind == "ln":
            gamma = g.const(rng.normal(1, 0.1, size=shape[-1]).astype(np.float32), "gamma")
            beta = g.const(rng.normal(0, 0.1, size=shape[-1]).astype(np.float32), "beta")
            cur = g.node("LayerNormalization", [cur, gamma, beta], shape, axis=-1, epsilon=1e-5)
        elif kind == "softmax":
            cur = g.node("Softmax", [cur], shape, axis=len(shape) - 1)
        elif kind == "attention" and len(shape) == 3 and shape[-1] % 64 == 0:
            heads, d = shape[-1] // int(rng.choice([32, 64])), 0
            d = shape[-1] // heads
            split = g.const(np.array([shape[0], shape[1], heads, d], dtype=np.int64), "split")
            merge = g.const(np.array(list(shape), dtype=np.int64), "merge")

            def heads_of(src):
                r = g.node("Reshape", [src, split], (shape[0], shape[1], heads, d))
                return g.node("Transpose", [r], (shape[0], heads, shape[1], d), perm=[0, 2, 1, 3])

            shared = cur if rng.random() < 0.7 else None     # Q, K, V from one input (widened) or from different ones
            q, k, v = (heads_of(linear(shared or str(rng.choice([p for p in pool if g.shapes[p] == shape] or [cur])),
                                       shape[-1])) for _ in range(3))
            kt = g.node("Transpose", [k], (shape[0], heads, d, shape[1]), perm=[0, 1, 3, 2])
            s = g.node("MatMul", [q, kt], (shape[0], heads, shape[1], shape[1]))
            s = g.node("Div", [s, g.const(np.float32(np.sqrt(d)), "sqrt_d")], g.shapes[s])
            pr = g.node("Softmax", [s], g.shapes[s], axis=3)
            ctx = g.node("MatMul", [pr, v], (shape[0], heads, shape[1], d))
            ctx = g.node("Transpose", [ctx], (shape[0], shape[1], heads, d), perm=[0, 2, 1, 3])
            cur = g.node("Reshape", [ctx, merge], shape)
        elif kind == "gemm" and len(shape) == 3:
            flat = g.const(np.array([shape[0] * shape[1], shape[2]], dtype=np.int64), "flat")
            back_n = int(rng.choice([32, 64]))
            two_d = g.node("Reshape", [cur, flat], (shape[0] * shape[1], shape[2]))
            w = g.const(rng.normal(0, 0.1, size=(back_n, shape[2])).astype(np.float32), "wt")   # [N, K]: transB
            c = g.const(rng.normal(0, 0.1, size=back_n).astype(np.float32), "c")
            y = g.node("Gemm", [two_d, w, c], (shape[0] * shape[1], back_n), transB=1)
            back = g.const(np.array([shape[0], shape[1], back_n], dtype=np.int64), "back")
            cur = g.node("Reshape", [y, back], (shape[0], shape[1], back_n))
        elif kind == "reuse":
            # a value with two readers: both branches are kept alive and meet again in an Add
            a = g.node("Relu", [cur], shape)
            b = g.node("Mul", [cur, g.const(np.float32(0.5), "half")], shape)
            cur = g.node("Add", [a, b], shape)
        pool.append(cur)
    graph = H.make_graph(g.nodes, f"random_{seed}", [H.make_tensor_value_info("x", T.FLOAT, list(x_shape))],
                         [H.make_tensor_value_info(cur, T.FLOAT, list(g.shapes[cur]))], initializer=g.inits)
    return H.make_model(graph, opset_imports=[H.make_opsetid("", 17)]), x_shape


def evaluate_with_oracle(model, x):
    """Node-by-node evaluation of the graph with the oracle's op restatements."""
    env = {t.name: np.asarray(t.array).reshape(t.dims) for t in model.graph.initializer}
    env["x"] = x
    for n in model.graph.node:
        a = {at.name: at.value for at in n.attribute}
        i = [env[k] for k in n.input]
        op = n.op_type
        if op == "MatMul":
            y = O.matmul(i[0], i[1])
        elif op == "Gemm":
            y = O.gemm(i[0], i[1], i[2] if len(i) > 2 else None, transB=int(a.get("transB", 0)))
        elif op in ("Add", "Mul", "Div"):
            y = getattr(O, op.lower())(i[0], i[1])
        elif op in ("Relu", "Gelu", "Tanh", "Sigmoid", "Softplus", "Abs", "Neg"):
            y = getattr(O, op.lower())(i[0])
        elif op == "LayerNormalization":
            y = O.layer_normalization(i[0], i[1], i[2], axis=-1, epsilon=float(a["epsilon"]))
        elif op == "Softmax":
            y = O.softmax(i[0], axis=int(a["axis"]))
        elif op == "Reshape":
            y = O.reshape(i[0], tuple(int(v) for v in i[1]))
        elif op == "Transpose":
            y = O.transpose(i[0], tuple(a["perm"]))
        else:
            raise AssertionError(op)
        env[n.output[0]] = y
    return env[model.graph.output[0].name]


SEEDS = list(range(40))


@pytest.mark.parametrize("seed", SEEDS)
def test_random_graph_fuses_and_expands(seed):
    model, _ = random_graph(seed)
    fused = donnx.ONNXModel(f"rg_fused_{seed}", model)
    plain = donnx.ONNXModel(f"rg_plain_{seed}", model, fuse=False)
    n_fused = sum(isinstance(n, dace.KernelCall) for n, _ in fused.expand().all_nodes_recursive())
    n_plain = sum(isinstance(n, dace.KernelCall) for n, _ in plain.expand().all_nodes_recursive())
    assert 1 <= n_fused <= n_plain
    for m in (fused, plain):     # everything became a kernel call or a view
        assert not any(isinstance(n, dace.LibraryNode) for n, _ in m.sdfg.all_nodes_recursive())


@pytest.mark.gpu
@pytest.mark.parametrize("seed", SEEDS)
def test_random_graph_values(seed):
    model, x_shape = random_graph(seed)
    x = np.random.default_rng(1000 + seed).normal(size=x_shape).astype(np.float32)
    expected = evaluate_with_oracle(model, x)
    print(f"random graph seed {seed}: {[n.op_type for n in model.graph.node]}", flush=True)
    fused = donnx.ONNXModel(f"rg_fused_{seed}", model)(x)
    plain = donnx.ONNXModel(f"rg_plain_{seed}", model, fuse=False)(x)
    assert rel_err(expected, plain) < FP32_REL_TOL
    assert rel_err(expected, fused) < FP32_REL_TOL

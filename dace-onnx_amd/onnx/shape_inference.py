"""Static shape and type inference for the supported ops.

The reference runs ``onnx.shape_inference`` (or the vendored symbolic inference,
``daceml/onnx/shape_inference/symbolic_shape_infer.py``) before it creates one
array per value (``daceml/onnx/onnx_importer.py:131-166``). Shapes on the hot
path are static, so this is the per-op rule set of the ONNX specification for
the ops that have an ``ONNX<Op>`` class here; value_info already present in the
model is kept and checked against.
"""
import typing

import numpy as np

from .proto import ModelProto, ValueInfoProto, TensorProto


class ShapeInferenceError(ValueError):
    pass


def _attrs(node):
    return {a.name: a.value for a in node.attribute}


def _conv_out(size, k, stride, dil, pad_lo, pad_hi):
    return (size + pad_lo + pad_hi - ((k - 1) * dil + 1)) // stride + 1


def slice_ranges(shape, starts, ends, axes=None, steps=None):
    """Per axis of ``shape``: (first index, step, number of elements) of an ONNX Slice, with the operator's
    clamping rules (negative indices count from the end, out-of-range bounds are clamped -- which is what
    Python slicing does; ``ends`` of INT64_MAX is the exporters' "to the end")."""
    rank = len(shape)
    starts, ends = [int(v) for v in starts], [int(v) for v in ends]
    axes = [int(v) for v in axes] if axes is not None else list(range(len(starts)))
    steps = [int(v) for v in steps] if steps is not None else [1] * len(starts)
    if not len(starts) == len(ends) == len(axes) == len(steps):
        raise ShapeInferenceError("Slice: starts, ends, axes and steps differ in length")
    out = [(0, 1, int(d)) for d in shape]
    for s, e, ax, st in zip(starts, ends, axes, steps):
        if not -rank <= ax < rank or st == 0:
            raise ShapeInferenceError(f"Slice: axis {ax} outside rank {rank}, or a zero step")
        selected = range(*slice(s, e, st).indices(int(shape[ax % rank])))
        out[ax % rank] = (selected.start, st, len(selected))
    return out


def _infer_node(node, shapes, types, constants):
    """Return [(shape, elem_type)] for each output of ``node``."""
    a = _attrs(node)
    ins = [shapes.get(i) for i in node.input]
    tys = [types.get(i) for i in node.input]
    op = node.op_type
    if any(s is None for s, name in zip(ins, node.input) if name != ""):
        missing = [n for n in node.input if n and n not in shapes]
        raise ShapeInferenceError(f"{op} node '{node.name}': no shape for input(s) {missing}")
    if op in ("Add", "Sub", "Mul", "Div", "Pow"):
        return [(tuple(np.broadcast_shapes(ins[0], ins[1])), tys[0])]
    if op in ("Relu", "Gelu", "Erf", "Sqrt", "Softmax", "LogSoftmax", "Identity", "Tanh", "Sigmoid", "Log", "Exp", "Softplus",
              "Reciprocal", "Neg", "Abs"):
        return [(ins[0], tys[0])]
    if op == "LayerNormalization":
        return [(ins[0], tys[0])]
    if op == "MatMul" or op == "MatMulInteger":
        A, B = ins[0], ins[1]
        if len(A) < 2 or len(B) < 2:
            raise ShapeInferenceError(f"{op} '{node.name}': 1-D operands are not supported")
        if A[-1] != B[-2]:
            raise ShapeInferenceError(f"{op} '{node.name}': inner dimensions {A[-1]} and {B[-2]} differ")
        batch = tuple(np.broadcast_shapes(A[:-2], B[:-2]))
        return [(batch + (A[-2], B[-1]), TensorProto.INT32 if op == "MatMulInteger" else tys[0])]
    if op == "Gemm":
        A, B = ins[0], ins[1]
        M = A[1] if a.get("transA", 0) else A[0]
        N = B[0] if a.get("transB", 0) else B[1]
        return [((M, N), tys[0])]
    if op == "Conv":
        X, W = ins[0], ins[1]
        nsp = len(X) - 2
        strides = a.get("strides") or [1] * nsp
        dil = a.get("dilations") or [1] * nsp
        auto_pad = a.get("auto_pad", "NOTSET")
        if isinstance(auto_pad, bytes):
            auto_pad = auto_pad.decode()
        out = []
        for i in range(nsp):
            if auto_pad in ("SAME_UPPER", "SAME_LOWER"):
                out.append(-(-X[2 + i] // strides[i]))
            else:
                pads = (a.get("pads") or [0] * (2 * nsp)) if auto_pad == "NOTSET" else [0] * (2 * nsp)
                out.append(_conv_out(X[2 + i], W[2 + i], strides[i], dil[i], pads[i], pads[i + nsp]))
        return [((X[0], W[0]) + tuple(out), tys[0])]
    if op == "Transpose":
        perm = a.get("perm") or list(reversed(range(len(ins[0]))))
        return [(tuple(ins[0][p] for p in perm), tys[0])]
    if op == "Reshape":
        if node.input[1] not in constants:
            # the shape is computed by other nodes (left in the graph when constants are not folded): the model
            # must then declare the result's shape, which is all the expansion needs (PureReshape reads the
            # output descriptor too, pure_implementations.py:497)
            declared = shapes.get(node.output[0])
            if declared is None or int(np.prod(declared)) != (int(np.prod(ins[0])) if len(ins[0]) else 1):
                raise ShapeInferenceError(f"Reshape '{node.name}': the shape input is not a constant initializer and "
                                          "the model declares no (matching) shape for the result")
            return [(tuple(declared), tys[0])]
        target = [int(v) for v in constants[node.input[1]].ravel()]
        total = int(np.prod(ins[0])) if len(ins[0]) else 1
        out = [ins[0][i] if v == 0 else v for i, v in enumerate(target)]
        if out.count(-1) > 1:
            raise ShapeInferenceError(f"Reshape '{node.name}': more than one -1 in {target}")
        if -1 in out:
            known = int(np.prod([v for v in out if v != -1])) if len(out) > 1 else 1
            out[out.index(-1)] = total // known if known else 0
        if int(np.prod(out)) != total:
            raise ShapeInferenceError(f"Reshape '{node.name}': cannot reshape {ins[0]} to {target}")
        return [(tuple(out), tys[0])]
    if op == "Pad":
        if node.input[1] not in constants:
            raise ShapeInferenceError(f"Pad '{node.name}': the pads input must be a constant initializer")
        pads = [int(v) for v in constants[node.input[1]].ravel()]
        rank = len(ins[0])
        if len(pads) != 2 * rank:
            raise ShapeInferenceError(f"Pad '{node.name}': {len(pads)} pads for a rank-{rank} input")
        return [(tuple(ins[0][i] + pads[i] + pads[i + rank] for i in range(rank)), tys[0])]
    if op == "Flatten":
        axis = a.get("axis", 1) % (len(ins[0]) + 1) if a.get("axis", 1) < 0 else a.get("axis", 1)
        return [((int(np.prod(ins[0][:axis])) if axis else 1, int(np.prod(ins[0][axis:]))), tys[0])]
    if op == "Squeeze":
        rank = len(ins[0])
        axes = [ax % rank for ax in a["axes"]] if a.get("axes") is not None else [i for i, d in enumerate(ins[0]) if d == 1]
        if any(ins[0][ax] != 1 for ax in axes):
            raise ShapeInferenceError(f"Squeeze '{node.name}': axes {axes} of {ins[0]} are not all of extent 1")
        return [(tuple(d for i, d in enumerate(ins[0]) if i not in axes), tys[0])]
    if op == "Unsqueeze":
        rank = len(ins[0]) + len(a["axes"])
        axes = sorted(ax % rank for ax in a["axes"])
        out = list(ins[0])
        for ax in axes:
            out.insert(ax, 1)
        return [(tuple(out), tys[0])]
    if op == "Cast":
        return [(ins[0], int(a["to"]))]
    if op == "Slice":
        idx = []
        for k in range(1, 5):
            name = node.input[k] if len(node.input) > k else ""
            if name and name not in constants:
                raise ShapeInferenceError(f"Slice '{node.name}': input '{name}' must be a constant initializer")
            idx.append([int(v) for v in constants[name].ravel()] if name else None)
        return [(tuple(c for _, _, c in slice_ranges(ins[0], *idx)), tys[0])]
    if op == "BatchNormalization":
        return [(ins[0], tys[0])] + [((ins[0][1], ), tys[0])] * (len(node.output) - 1)
    if op == "GlobalAveragePool":
        return [(tuple(ins[0][:2]) + (1, ) * (len(ins[0]) - 2), tys[0])]
    if op == "MaxPool":
        X = ins[0]
        nsp = len(X) - 2
        kernel = a.get("kernel_shape")
        strides = a.get("strides") or [1] * nsp
        dil = a.get("dilations") or [1] * nsp
        auto_pad = a.get("auto_pad", "NOTSET")
        auto_pad = auto_pad.decode() if isinstance(auto_pad, bytes) else auto_pad
        if a.get("ceil_mode", 0):
            raise ShapeInferenceError(f"MaxPool '{node.name}': ceil_mode is not supported")
        out = []
        for i in range(nsp):
            if auto_pad in ("SAME_UPPER", "SAME_LOWER"):
                out.append(-(-X[2 + i] // strides[i]))
            else:
                pads = (a.get("pads") or [0] * (2 * nsp)) if auto_pad == "NOTSET" else [0] * (2 * nsp)
                out.append(_conv_out(X[2 + i], kernel[i], strides[i], dil[i], pads[i], pads[i + nsp]))
        return [((X[0], X[1]) + tuple(out), tys[0])] + [((X[0], X[1]) + tuple(out), TensorProto.INT64)] * (len(node.output) - 1)
    if op == "Einsum":
        eq = a["equation"].decode() if isinstance(a["equation"], bytes) else a["equation"]
        eq = eq.replace(" ", "")
        if "..." in eq or "->" not in eq:
            raise ShapeInferenceError(f"Einsum '{node.name}': only explicit equations without ellipsis ('{eq}')")
        lhs, out = eq.split("->")
        size = {}
        for term, shp in zip(lhs.split(","), ins):
            if len(term) != len(shp):
                raise ShapeInferenceError(f"Einsum '{node.name}': term '{term}' does not match a rank-{len(shp)} input")
            size.update(zip(term, shp))
        return [(tuple(size[c] for c in out), tys[0])]
    if op == "Sum":
        return [(tuple(np.broadcast_shapes(*ins)), tys[0])]
    if op in ("ReduceMean", "ReduceSum", "ReduceMax", "ReduceMin"):
        axes = a.get("axes") or list(range(len(ins[0])))
        axes = [ax % len(ins[0]) for ax in axes]
        keep = a.get("keepdims", 1)
        out = [1 if i in axes else s for i, s in enumerate(ins[0]) if keep or i not in axes]
        return [(tuple(out), tys[0])]
    raise ShapeInferenceError(f"no shape rule for op '{op}' (node '{node.name}')")


def infer_shapes(model: ModelProto) -> ModelProto:
    """Fill ``graph.value_info`` for every intermediate value (in place; returns the model)."""
    g = model.graph
    shapes: typing.Dict[str, tuple] = {}
    types: typing.Dict[str, int] = {}
    constants = {}
    for t in g.initializer:
        shapes[t.name] = tuple(t.dims)
        types[t.name] = t.data_type
        constants[t.name] = t.array
    for v in list(g.input) + list(g.value_info) + list(g.output):
        if v.shape is not None and all(isinstance(d, int) for d in v.shape):
            shapes.setdefault(v.name, tuple(v.shape))
            types.setdefault(v.name, v.elem_type)
    known_vi = {v.name for v in g.value_info} | {v.name for v in g.output} | {v.name for v in g.input}
    for node in g.node:
        results = _infer_node(node, shapes, types, constants)
        for out_name, (shape, ty) in zip(node.output, results):
            if out_name in shapes and tuple(shapes[out_name]) != tuple(shape):
                raise ShapeInferenceError(
                    f"{node.op_type} '{node.name}': inferred shape {shape} for '{out_name}' "
                    f"contradicts the declared shape {shapes[out_name]}")
            shapes[out_name], types[out_name] = tuple(shape), ty
            if out_name not in known_vi:
                g.value_info.append(ValueInfoProto(out_name, ty, list(shape)))
                known_vi.add(out_name)
    # an output (or intermediate) declared without a shape, or with symbolic dimensions -- exporters write those
    # when their own inference gives up on computed pads / targets -- takes the inferred static shape
    for v in list(g.output) + list(g.value_info):
        static = v.shape is not None and all(isinstance(d, int) for d in v.shape)
        if not static and v.name in shapes:
            v.shape, v.elem_type = list(shapes[v.name]), types[v.name]
    return model

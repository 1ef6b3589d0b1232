"""Constant folding: nodes whose inputs are all known are removed and their outputs become weights.

The reference's ``ConstantFolding`` transformation (``daceml/transformation/constant_folding.py:48-216``)
matches any ONNX node whose inputs are all weights of the imported model -- or a ``Shape`` node whose
input has a static shape (``:86-97``) -- evaluates it through ONNX Runtime and stores the result as a new
weight. ``ONNXModel`` applies it when ``fold_constants`` is set (``onnx_importer.py:300-306``). It is what
turns the exporter's shape arithmetic (``Constant -> Unsqueeze -> Concat -> Reshape`` with
``do_constant_folding=False``) into plain constant shapes.

Here the same rule runs on the ``ModelProto`` before the graph is built, and nodes are evaluated with
numpy, for the operators that exporters use in such constant subgraphs. Two deliberate differences:

* an operator without a numpy rule below is left in the graph (the reference can evaluate anything ONNX
  Runtime can);
* ``Transpose`` of a large weight (``nn.Linear`` exports its ``[out, in]`` weight behind one) is left in
  the graph: the fusion pass turns it into GEMM operand strides, which costs no copy and keeps the weight
  tied to the module parameter it came from.
"""
import copy
import typing

import numpy as np

from ..onnx import proto
from ..onnx.proto import ModelProto

#: a Transpose / Reshape / Identity result larger than this stays a node (see the module docstring)
MAX_FOLDED_VIEW_ELEMENTS = 4096


def _attrs(node):
    return {a.name: a.value for a in node.attribute}


def _axes(a, ins, idx):
    """``axes`` as an attribute (up to opset 12) or as input ``idx`` (opset 13 on)."""
    if a.get("axes") is not None:
        return [int(v) for v in a["axes"]]
    if len(ins) > idx and ins[idx] is not None:
        return [int(v) for v in np.asarray(ins[idx]).reshape(-1)]
    return None


def _evaluate(node, ins: typing.List[typing.Optional[np.ndarray]]) -> typing.Optional[typing.List[np.ndarray]]:
    """Outputs of ``node`` for constant inputs, or None when there is no rule for it."""
    op, a = node.op_type, _attrs(node)
    x = ins[0] if ins else None
    if op == "Identity":
        return [x]
    if op == "Unsqueeze":
        axes = _axes(a, ins, 1)
        rank = x.ndim + len(axes)       # negative axes count from the end of the output
        out = x
        for ax in sorted(ax + rank if ax < 0 else ax for ax in axes):
            out = np.expand_dims(out, ax)
        return [out]
    if op == "Squeeze":
        axes = _axes(a, ins, 1)
        return [np.squeeze(x, axis=tuple(axes) if axes is not None else None)]
    if op == "Concat":
        return [np.concatenate([np.asarray(v) for v in ins], axis=int(a["axis"]))]
    if op == "Cast":
        return [x.astype(proto.tensor_dtype_to_np_dtype(int(a["to"])))]
    if op == "Gather":
        return [np.take(x, np.asarray(ins[1]).astype(np.int64), axis=int(a.get("axis", 0)))]
    if op == "Slice":
        starts, ends = (np.asarray(v).reshape(-1) for v in ins[1:3])
        axes = np.asarray(ins[3]).reshape(-1) if len(ins) > 3 and ins[3] is not None else np.arange(len(starts))
        steps = np.asarray(ins[4]).reshape(-1) if len(ins) > 4 and ins[4] is not None else np.ones(len(starts), np.int64)
        index = [slice(None)] * x.ndim
        for s, e, ax, st in zip(starts, ends, axes, steps):
            index[int(ax)] = slice(int(s), int(e), int(st))     # numpy clamps out-of-range bounds as ONNX does
        return [x[tuple(index)]]
    if op in ("Add", "Sub", "Mul", "Div"):
        y = ins[1]
        if op == "Div" and np.issubdtype(x.dtype, np.integer):
            return [np.trunc(np.true_divide(x, y)).astype(x.dtype)]   # C semantics: truncation toward zero
        return [{"Add": np.add, "Sub": np.subtract, "Mul": np.multiply, "Div": np.divide}[op](x, y).astype(x.dtype)]
    if op == "Neg":
        return [np.negative(x)]
    if op == "Sqrt":
        return [np.sqrt(x)]
    if op == "Reshape":
        target = [int(v) for v in np.asarray(ins[1]).reshape(-1)]
        target = [x.shape[i] if d == 0 else d for i, d in enumerate(target)]
        return [x.reshape(target)] if x.size <= MAX_FOLDED_VIEW_ELEMENTS else None
    if op == "Transpose":
        perm = a.get("perm")
        return [np.ascontiguousarray(np.transpose(x, perm))] if x.size <= MAX_FOLDED_VIEW_ELEMENTS else None
    if op == "ConstantOfShape":
        value = a.get("value")
        fill = np.asarray(value.array).reshape(-1)[0] if value is not None else np.float32(0)
        return [np.full([int(v) for v in np.asarray(x).reshape(-1)], fill)]
    if op == "Range":
        return [np.arange(ins[0].item(), ins[1].item(), ins[2].item()).astype(ins[0].dtype)]
    return None


def fold_constants(model: ModelProto) -> ModelProto:
    """Returns a model in which every node with known inputs (and a rule above) has been replaced by an
    initializer, in graph order (so chains fold in one pass); ``Shape`` of a value with a static shape
    counts as known. Initializers that nothing reads any more are dropped unless the graph lists them as
    inputs (the module's parameters under ``keep_initializers_as_inputs``). The caller's model is not
    modified."""
    graph = model.graph
    consts = {t.name: np.asarray(t.array).reshape(t.dims) for t in graph.initializer}
    listed = {v.name for v in graph.input}
    static_shapes = {v.name: v.shape for v in list(graph.input) + list(graph.value_info) + list(graph.output)
                     if v.shape is not None and all(isinstance(d, int) for d in v.shape)}
    kept, folded = [], {}
    for node in graph.node:
        outs = None
        if node.op_type == "Shape" and len(node.input) == 1:
            src = node.input[0]
            shape = consts[src].shape if src in consts else static_shapes.get(src)
            if shape is not None:
                outs = [np.asarray(shape, dtype=np.int64)]
        elif node.input and all(name == "" or name in consts for name in node.input):
            outs = _evaluate(node, [consts[name] if name else None for name in node.input])
        if outs is None or len(outs) != len(node.output):
            kept.append(node)
            continue
        for name, value in zip(node.output, outs):
            consts[name] = folded[name] = np.asarray(value)
    if not folded:
        return model
    used = {name for node in kept for name in node.input} | {o.name for o in graph.output}
    model = copy.copy(model)
    model.graph = copy.copy(graph)
    model.graph.node = kept
    model.graph.initializer = [t for t in graph.initializer if t.name in used or t.name in listed] + \
        [proto.numpy_helper.from_array(v, name=k) for k, v in folded.items() if k in used]
    # value_info of a folded value would contradict nothing, but is dead weight
    model.graph.value_info = [v for v in graph.value_info if v.name not in folded or v.name in used]
    return model

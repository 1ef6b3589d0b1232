"""ONNX operator schemas for the ops on the hot path.

The reference builds ``ONNXSchema`` objects from ``onnx.defs`` at import time
(``daceml/onnx/schema.py``, ``daceml/onnx/nodes/onnx_op.py:478-507``). The
``onnx`` package is not a dependency here, so the schemas of the supported ops
are written out: connector names, parameter kinds, attributes with defaults and
type constraints are those of the ONNX operator specification (opset 12 for the
ops the reference generates; LayerNormalization is opset 17 and Gelu opset 20,
which the reference does not have).
"""
import enum
import typing

from .. import sdfg as dace


class ONNXParameterType(enum.Enum):
    Single = 0
    Optional = 1
    Variadic = 2


class ONNXAttributeType(enum.Enum):
    Int = 1
    Float = 2
    String = 3
    Ints = 4
    Floats = 5
    Strings = 6
    Tensor = 7


class ONNXParameter:
    def __init__(self, name, type_str, param_type=ONNXParameterType.Single, homogeneous=True):
        self.name, self.type_str, self.param_type, self.homogeneous = name, type_str, param_type, homogeneous


class ONNXAttribute:
    def __init__(self, name, attribute_type, default_value=None, required=False):
        self.name, self.attribute_type, self.default_value, self.required = \
            name, attribute_type, default_value, required


class ONNXTypeConstraint:
    def __init__(self, type_str, types):
        self.type_str, self.types = type_str, list(types)


class ONNXSchema:
    def __init__(self, name, since_version, inputs, outputs, attributes=(), type_constraints=(), doc=""):
        self.name = name
        self.since_version = since_version
        self.inputs: typing.List[ONNXParameter] = list(inputs)
        self.outputs: typing.List[ONNXParameter] = list(outputs)
        self.attributes = {a.name: a for a in attributes}
        self.type_constraints = {c.type_str: c for c in type_constraints}
        self.doc = doc

    def non_variadic_inputs(self):
        return [i.name for i in self.inputs if i.param_type != ONNXParameterType.Variadic]

    def variadic_inputs(self):
        return [i.name for i in self.inputs if i.param_type == ONNXParameterType.Variadic]

    def non_variadic_outputs(self):
        return [i.name for i in self.outputs if i.param_type != ONNXParameterType.Variadic]

    def variadic_outputs(self):
        return [i.name for i in self.outputs if i.param_type == ONNXParameterType.Variadic]


_S, _O = ONNXParameterType.Single, ONNXParameterType.Optional
_A = ONNXAttributeType
_FLOATS = [dace.float16, dace.float32, dace.float64]
_NUMERIC = _FLOATS + [dace.int32, dace.int64, dace.uint8, dace.int8, dace.int16]
_ANY = _NUMERIC + [dace.bool_]


def _unary(name, version, in_name, out_name, types=_FLOATS, attributes=(), doc=""):
    return ONNXSchema(name, version, [ONNXParameter(in_name, "T")], [ONNXParameter(out_name, "T")],
                      attributes, [ONNXTypeConstraint("T", types)], doc)


def _binary(name, version, doc=""):
    return ONNXSchema(name, version, [ONNXParameter("A", "T"), ONNXParameter("B", "T")],
                      [ONNXParameter("C", "T")], (), [ONNXTypeConstraint("T", _NUMERIC)], doc)


SCHEMAS: typing.List[ONNXSchema] = [
    ONNXSchema("MatMul", 9, [ONNXParameter("A", "T"), ONNXParameter("B", "T")], [ONNXParameter("Y", "T")],
               (), [ONNXTypeConstraint("T", _FLOATS + [dace.int32, dace.int64])],
               "Matrix product that behaves like numpy.matmul."),
    ONNXSchema("Gemm", 11,
               [ONNXParameter("A", "T"), ONNXParameter("B", "T"), ONNXParameter("C", "T", _O)],
               [ONNXParameter("Y", "T")],
               [ONNXAttribute("alpha", _A.Float, 1.0), ONNXAttribute("beta", _A.Float, 1.0),
                ONNXAttribute("transA", _A.Int, 0), ONNXAttribute("transB", _A.Int, 0)],
               [ONNXTypeConstraint("T", _FLOATS + [dace.int32, dace.int64])],
               "Y = alpha * A' * B' + beta * C."),
    ONNXSchema("Conv", 11,
               [ONNXParameter("X", "T"), ONNXParameter("W", "T"), ONNXParameter("B", "T", _O)],
               [ONNXParameter("Y", "T")],
               [ONNXAttribute("auto_pad", _A.String, "NOTSET"), ONNXAttribute("dilations", _A.Ints),
                ONNXAttribute("group", _A.Int, 1), ONNXAttribute("kernel_shape", _A.Ints),
                ONNXAttribute("pads", _A.Ints), ONNXAttribute("strides", _A.Ints)],
               [ONNXTypeConstraint("T", _FLOATS)], "N-D convolution (cross-correlation)."),
    ONNXSchema("MatMulInteger", 10,
               [ONNXParameter("A", "T1"), ONNXParameter("B", "T2"),
                ONNXParameter("a_zero_point", "T1", _O), ONNXParameter("b_zero_point", "T2", _O)],
               [ONNXParameter("Y", "T3")], (),
               [ONNXTypeConstraint("T1", [dace.int8, dace.uint8]),
                ONNXTypeConstraint("T2", [dace.int8, dace.uint8]),
                ONNXTypeConstraint("T3", [dace.int32])],
               "Integer matrix product with zero points, int32 result."),
    _unary("Softmax", 11, "input", "output", attributes=[ONNXAttribute("axis", _A.Int, 1)],
           doc="Softmax along `axis`."),
    ONNXSchema("LayerNormalization", 17,
               [ONNXParameter("X", "T"), ONNXParameter("Scale", "T"), ONNXParameter("B", "T", _O)],
               [ONNXParameter("Y", "T"), ONNXParameter("Mean", "U", _O), ONNXParameter("InvStdDev", "U", _O)],
               [ONNXAttribute("axis", _A.Int, -1), ONNXAttribute("epsilon", _A.Float, 1e-5),
                ONNXAttribute("stash_type", _A.Int, 1)],
               [ONNXTypeConstraint("T", _FLOATS), ONNXTypeConstraint("U", [dace.float32])],
               "Layer normalization over the trailing dimensions starting at `axis`."),
    _binary("Add", 7), _binary("Sub", 7), _binary("Mul", 7), _binary("Div", 7),
    _unary("Relu", 6, "X", "Y"),
    _unary("Gelu", 20, "X", "Y", attributes=[ONNXAttribute("approximate", _A.String, "none")]),
    _unary("Erf", 9, "input", "output", types=_NUMERIC),
    _unary("Sqrt", 6, "X", "Y"),
    _unary("Log", 6, "input", "output"), _unary("Tanh", 6, "input", "output"), _unary("Exp", 6, "input", "output"),
    _unary("Sigmoid", 6, "X", "Y"), _unary("Softplus", 1, "X", "Y"), _unary("Reciprocal", 6, "X", "Y"),
    _unary("Neg", 6, "X", "Y", types=_FLOATS + [dace.int32, dace.int64, dace.int8, dace.int16]),
    _unary("Abs", 6, "X", "Y", types=_NUMERIC),
    ONNXSchema("Reshape", 5, [ONNXParameter("data", "T"), ONNXParameter("shape", "tensor(int64)")],
               [ONNXParameter("reshaped", "T")], (),
               [ONNXTypeConstraint("T", _ANY), ONNXTypeConstraint("tensor(int64)", [dace.int64])]),
    _unary("Transpose", 1, "data", "transposed", types=_ANY, attributes=[ONNXAttribute("perm", _A.Ints)]),
    _unary("Flatten", 11, "input", "output", types=_ANY, attributes=[ONNXAttribute("axis", _A.Int, 1)]),
    _unary("Identity", 1, "input", "output", types=_ANY),
    _unary("Squeeze", 11, "data", "squeezed", types=_ANY, attributes=[ONNXAttribute("axes", _A.Ints)]),
    _unary("Unsqueeze", 11, "data", "expanded", types=_ANY, attributes=[ONNXAttribute("axes", _A.Ints, required=True)]),
    # Pad only ever runs folded into the Conv that reads it (transformation/fusion.py, the reference's PadConvFusion)
    ONNXSchema("Pad", 11,
               [ONNXParameter("data", "T"), ONNXParameter("pads", "tensor(int64)"), ONNXParameter("constant_value", "T", _O)],
               [ONNXParameter("output", "T")], [ONNXAttribute("mode", _A.String, "constant")],
               [ONNXTypeConstraint("T", _NUMERIC), ONNXTypeConstraint("tensor(int64)", [dace.int64])],
               "Pad `data` by `pads` = [begin_0, ..., begin_n, end_0, ..., end_n]."),
    # Not an ONNX operator: the node the fusion pass puts in place of MatMul -> scale -> Softmax -> MatMul.
    ONNXSchema("FusedAttention", 1,
               [ONNXParameter("Q", "T"), ONNXParameter("K", "T"), ONNXParameter("V", "T")], [ONNXParameter("O", "T")],
               [ONNXAttribute("scale", _A.Float, 1.0)], [ONNXTypeConstraint("T", [dace.float32])],
               "softmax(scale * Q K^T) V per batch entry; Q, O are [..., Sq, D], K, V are [..., Sk, D]."),
    # Not an ONNX operator: a group of elementwise nodes merged by the fusion pass into one launch.
    ONNXSchema("FusedElementwise", 1, [ONNXParameter("X", "T", ONNXParameterType.Variadic)], [ONNXParameter("Y", "T")],
               [ONNXAttribute("program", _A.Ints), ONNXAttribute("immediates", _A.Floats), ONNXAttribute("kinds", _A.Ints)],
               [ONNXTypeConstraint("T", [dace.float32])],
               "Y = program(X__0, X__1, ...): instructions, immediates and operand kinds as in mi355x_eltwise_program_f32."),
    ONNXSchema("Pow", 12, [ONNXParameter("X", "T"), ONNXParameter("Y", "T1")], [ONNXParameter("Z", "T")], (),
               [ONNXTypeConstraint("T", _FLOATS + [dace.int32, dace.int64]), ONNXTypeConstraint("T1", _NUMERIC)]),
] + [
    ONNXSchema(name, 11, [ONNXParameter("data", "T")], [ONNXParameter("reduced", "T")],
               [ONNXAttribute("axes", _A.Ints), ONNXAttribute("keepdims", _A.Int, 1)],
               [ONNXTypeConstraint("T", _FLOATS + [dace.int32, dace.int64])])
    for name in ("ReduceMean", "ReduceSum", "ReduceMax", "ReduceMin")
] + [
    _unary("LogSoftmax", 11, "input", "output", attributes=[ONNXAttribute("axis", _A.Int, 1)],
           doc="Log of the softmax along `axis`."),
    ONNXSchema("Cast", 9, [ONNXParameter("input", "T1")], [ONNXParameter("output", "T2")],
               [ONNXAttribute("to", _A.Int, required=True)],
               [ONNXTypeConstraint("T1", _ANY), ONNXTypeConstraint("T2", _ANY)], "Elementwise conversion to the type `to`."),
    ONNXSchema("Slice", 11,
               [ONNXParameter("data", "T"), ONNXParameter("starts", "Tind"), ONNXParameter("ends", "Tind"),
                ONNXParameter("axes", "Tind", _O), ONNXParameter("steps", "Tind", _O)],
               [ONNXParameter("output", "T")], (),
               [ONNXTypeConstraint("T", _ANY), ONNXTypeConstraint("Tind", [dace.int32, dace.int64])],
               "data[starts:ends:steps] along `axes` (numpy slicing semantics, bounds clamped)."),
    ONNXSchema("Einsum", 12, [ONNXParameter("Inputs", "T", ONNXParameterType.Variadic)], [ONNXParameter("Output", "T")],
               [ONNXAttribute("equation", _A.String, required=True)],
               [ONNXTypeConstraint("T", _FLOATS + [dace.int32, dace.int64])], "Einstein summation."),
    ONNXSchema("MaxPool", 12, [ONNXParameter("X", "T")], [ONNXParameter("Y", "T"), ONNXParameter("Indices", "I", _O)],
               [ONNXAttribute("auto_pad", _A.String, "NOTSET"), ONNXAttribute("ceil_mode", _A.Int, 0),
                ONNXAttribute("dilations", _A.Ints), ONNXAttribute("kernel_shape", _A.Ints, required=True),
                ONNXAttribute("pads", _A.Ints), ONNXAttribute("storage_order", _A.Int, 0), ONNXAttribute("strides", _A.Ints)],
               [ONNXTypeConstraint("T", _FLOATS + [dace.int8, dace.uint8]), ONNXTypeConstraint("I", [dace.int64])],
               "Max pooling over sliding windows."),
    _unary("GlobalAveragePool", 1, "X", "Y", doc="Mean over the spatial axes."),
    ONNXSchema("BatchNormalization", 9,
               [ONNXParameter("X", "T"), ONNXParameter("scale", "T"), ONNXParameter("B", "T"), ONNXParameter("in_mean", "T"),
                ONNXParameter("in_var", "T")],
               [ONNXParameter("Y", "T"), ONNXParameter("out_mean", "T", _O), ONNXParameter("out_var", "T", _O),
                ONNXParameter("saved_mean", "T", _O), ONNXParameter("saved_var", "T", _O)],
               [ONNXAttribute("epsilon", _A.Float, 1e-5), ONNXAttribute("momentum", _A.Float, 0.9)],
               [ONNXTypeConstraint("T", _FLOATS)], "Batch normalization. ONNX names the statistics `mean` / `var` on both sides; as in the reference "
               "(onnx_op.py:499-508) the inputs are `in_mean` / `in_var` and the outputs `out_mean` / `out_var`."),
    ONNXSchema("Sum", 8, [ONNXParameter("data_0", "T", ONNXParameterType.Variadic)], [ONNXParameter("sum", "T")], (),
               [ONNXTypeConstraint("T", _FLOATS)], "Elementwise sum of the inputs."),
]

SCHEMAS_BY_NAME = {s.name: s for s in SCHEMAS}

"""ONNX library nodes: one ``ONNX<Op>`` class per schema, with the reference's
construction, validation and implementation-binding behaviour
(``daceml/onnx/nodes/onnx_op.py:84-415`` ONNXOp and validate, ``:494-694`` class
generation and binding, ``:418-475`` the Python-frontend call form).
"""
import itertools
import logging
import typing

from ...sdfg import SDFG, SDFGState, LibraryNode, MultiConnectorEdge
from ..schema import ONNXSchema, ONNXParameterType, SCHEMAS
from .node_utils import parse_variadic_param

log = logging.getLogger(__name__)


def get_missing_arguments_message(function_name, missing_arguments, argument_type):
    names = list(map(lambda x: "'" + x + "'", missing_arguments))
    if len(missing_arguments) == 1:
        arglist = names[0]
    else:
        arglist = ", ".join(names[:-1]) + ", and " + names[-1]
    return "{function_name} missing {num_missing} required {argument_type}{s}: {arglist}".format(
        function_name=function_name, num_missing=len(missing_arguments), argument_type=argument_type,
        s='' if len(missing_arguments) == 1 else 's', arglist=arglist)


def _is_private(connector: str) -> bool:
    return connector.startswith("_")


class ExpansionRefused(NotImplementedError):
    """No implementation available in this build can expand the node.

    In the reference a refused expansion falls back to ONNX Runtime
    (``onnx_op.py:668-680``). ONNX Runtime is not part of this build and there is
    no host implementation to fall back to, so the fallback raises instead of
    silently computing somewhere else.
    """


class ONNXOp(LibraryNode):
    """Abstract superclass of all ONNX ops; use the generated subclasses."""

    implementations: typing.Dict[str, typing.Any] = {}
    default_implementation = None
    schema: ONNXSchema = None

    def __new__(cls, *args, **kwargs):
        # Python-frontend call form, e.g. donnx.ONNXConv(X=x, W=w, Y=y, strides=[2, 2]):
        # connector names appear as keyword arguments (onnx_op.py:420-475).
        if cls.schema is not None and not args and "name" not in kwargs:
            conns = set(cls.schema.non_variadic_inputs()) | set(cls.schema.non_variadic_outputs())
            if conns & set(kwargs):
                from .frontend import call_onnx_op
                return call_onnx_op(cls, **kwargs)
        return super().__new__(cls)

    # ---- edges in schema order (onnx_op.py:107-189) ----------------------------------
    def iter_outputs_in_onnx_order(self, state: SDFGState) -> typing.List[MultiConnectorEdge]:
        return self._iter_params_in_onnx_order(state, inputs=False)

    def iter_inputs_in_onnx_order(self, state: SDFGState) -> typing.List[MultiConnectorEdge]:
        return self._iter_params_in_onnx_order(state, inputs=True)

    def _iter_params_in_onnx_order(self, state, inputs=False):
        parameters = list(self.schema.inputs if inputs else self.schema.outputs)
        if len(parameters) == 0:
            return []
        if parameters[-1].param_type == ONNXParameterType.Variadic:
            name = parameters[-1].name
            names = itertools.chain([p.name for p in parameters[:-1]],
                                    (name + "__" + str(i) for i in itertools.count()))
        else:
            names = [p.name for p in parameters]
        edges = state.in_edges(self) if inputs else state.out_edges(self)
        conn_to_edge = {(e.dst_conn if inputs else e.src_conn): e for e in edges}
        out = []
        for n in itertools.islice(names, len(parameters) + len(edges)):
            if n in conn_to_edge:
                out.append(conn_to_edge[n])
        return out

    def iter_edges(self, state: SDFGState):
        """(edge, is_input) pairs ordered as the schema orders its parameters."""
        def get_idx(parameters, name):
            number = 0
            if '__' in name:
                name, number = parse_variadic_param(name)
            matched = [i for i, param in enumerate(parameters) if param.name == name]
            if len(matched) != 1:
                raise ValueError("Found {} connectors with name '{}', expected to find exactly one".format(
                    len(matched), name))
            return matched[0] + number

        # connectors with a leading underscore are private to an implementation (operands
        # folded in by the fusion pass); they are not schema parameters
        sorted_in = sorted((e for e in state.in_edges(self) if not _is_private(e.dst_conn)),
                           key=lambda e: get_idx(self.schema.inputs, e.dst_conn))
        sorted_out = sorted((e for e in state.out_edges(self) if not _is_private(e.src_conn)),
                            key=lambda e: get_idx(self.schema.outputs, e.src_conn))
        return itertools.chain(zip(sorted_in, itertools.repeat(True)), zip(sorted_out, itertools.repeat(False)))

    # ---- validation (onnx_op.py:197-415) ------------------------------------------------
    def validate(self, sdfg: SDFG, state: SDFGState):
        in_edges = state.in_edges(self)
        out_edges = state.out_edges(self)

        all_connectors = {e.dst_conn for e in in_edges}.union(e.src_conn for e in out_edges)
        if None in all_connectors:
            raise ValueError("Edges to ONNX Ops must not have connector None")
        in_edges = [e for e in in_edges if not _is_private(e.dst_conn)]
        out_edges = [e for e in out_edges if not _is_private(e.src_conn)]

        known_inputs = {inp.name for inp in self.schema.inputs}
        known_outputs = {outp.name for outp in self.schema.outputs}
        passed_inputs = {e.dst_conn for e in in_edges if '__' not in e.dst_conn}
        passed_outputs = {e.src_conn for e in out_edges if '__' not in e.src_conn}

        unknown_inputs = passed_inputs.difference(known_inputs)
        if len(unknown_inputs) > 0:
            raise TypeError("Got an unexpected argument '{}'".format(sorted(unknown_inputs)[0]))
        unknown_outputs = passed_outputs.difference(known_outputs)
        if len(unknown_outputs) > 0:
            raise TypeError("Got an unexpected argument '{}'".format(sorted(unknown_outputs)[0]))

        for edge, is_input in self.iter_edges(state):
            conn_name = edge.dst_conn if is_input else edge.src_conn
            if conn_name not in (self.in_connectors if is_input else self.out_connectors):
                raise ValueError("Memlet {} leading to nonexistent {} connector '{}'".format(
                    edge.data, "input" if is_input else "output", conn_name))

        required_inputs = {i.name for i in self.schema.inputs if i.param_type == ONNXParameterType.Single}
        missing_inputs = required_inputs.difference(passed_inputs)
        if len(missing_inputs) > 0:
            raise ValueError(get_missing_arguments_message(self.schema.name, sorted(missing_inputs), "input"))
        required_outputs = {o.name for o in self.schema.outputs if o.param_type == ONNXParameterType.Single}
        missing_outputs = required_outputs.difference(passed_outputs)
        if len(missing_outputs) > 0:
            raise ValueError(get_missing_arguments_message(self.schema.name, sorted(missing_outputs), "output"))

        for is_input, edges, params in ((True, in_edges, self.schema.inputs), (False, out_edges, self.schema.outputs)):
            variadic = {p.name for p in params if p.param_type == ONNXParameterType.Variadic}
            passed = {(e.dst_conn if is_input else e.src_conn) for e in edges}
            passed = {c for c in passed if '__' in c}
            seen = set()
            for param in passed:
                name, number = parse_variadic_param(param)
                if name not in variadic:
                    raise ValueError("Got an unexpected variadic argument '{}'".format(param))
                if number in seen:
                    raise ValueError("Got two variadic {} with index {}, expected at most one".format(
                        "inputs" if is_input else "outputs", number))
                seen.add(number)
            for i in range(len(seen)):
                if i not in seen:
                    raise ValueError("Since {} variadic {} were passed, expected variadic parameter with number {}"
                                     .format(len(seen), "inputs" if is_input else "outputs", i))

        # type constraints must solve
        assigned_params = {}
        for edge, is_input in self.iter_edges(state):
            conn_name = edge.dst_conn if is_input else edge.src_conn
            parsed_name = parse_variadic_param(conn_name)[0] if '__' in conn_name else conn_name
            matching = [p for p in (self.schema.inputs if is_input else self.schema.outputs) if p.name == parsed_name]
            if len(matching) != 1:
                raise ValueError("Expected to find one {} parameter in schema with name '{}', but found {}".format(
                    "input" if is_input else "output", parsed_name, len(matching)))
            matched = matching[0]
            if '__' in conn_name and matched.param_type != ONNXParameterType.Variadic:
                raise ValueError("Got variadic argument '{}' for non-variadic parameter '{}'."
                                 " Ensure that non-variadic args do not contain '__'".format(conn_name, matched.name))
            edge_dtype = sdfg.arrays[edge.data.data].dtype
            if matched.type_str in assigned_params and assigned_params[matched.type_str] != edge_dtype:
                raise ValueError("Could not solve type constraints;"
                                 " excepted type '{expected}' for {param_type} '{conn_name}', got type '{actual}'".format(
                                     expected=assigned_params[matched.type_str],
                                     param_type="input" if is_input else "output",
                                     conn_name=matched.name, actual=edge_dtype))
            cons = self.schema.type_constraints[matched.type_str]
            if edge_dtype not in cons.types:
                raise ValueError("Expected type in '{possible}' for {param_type} '{conn_name}', got type '{actual}'".format(
                    possible=cons.types, param_type="input" if is_input else "output",
                    conn_name=matched.name, actual=edge_dtype))
            assigned_params[matched.type_str] = edge_dtype

        for name, attr in self.schema.attributes.items():
            if attr.required and getattr(self, name) is None:
                raise ValueError("Expected value for required attribute '{}', got None".format(name))


# ------------------------------------------------------------------------------------
# implementation binding


class ExpandTransformation:
    """Holds one way of expanding a library node (``dace`` ExpandTransformation)."""
    environments: typing.List[typing.Any] = []

    @classmethod
    def expansion(cls, node, state, sdfg):
        raise NotImplementedError


def expand_node(node, state, sdfg):
    """The ``"onnxruntime"`` expansion (``daceml/onnx/nodes/node_codegen.py:321``).

    ONNX Runtime is not part of this build: every supported configuration is
    covered by the ``"mi355x"`` kernels and anything else is an error, never a
    silent host computation.
    """
    raise ExpansionRefused(
        f'library node "{node.label}" ({node.schema.name}) cannot be expanded: the "onnxruntime" '
        f"implementation is not available in this build and no other implementation accepted the node")


def _make_ort_expansion():
    class Expansion(ExpandTransformation):
        environments = []

        @classmethod
        def expansion(cls, node, state, sdfg):
            return expand_node(node, state, sdfg)

    return Expansion


def bind_implementation(op_name: str, implementation_name: str, impl) -> bool:
    """Make ``impl`` (an ``ONNXForward`` subclass) selectable on ``ONNX<op_name>``.

    Same wrapper as ``onnx_op.py:652-683``: validate, ask
    ``forward_can_be_applied``, call ``forward``, otherwise fall back to the
    ``"onnxruntime"`` expansion. Unlike the reference's import-time loop this can
    be called at any time, so implementations defined outside the package are
    bound when they are registered.
    """
    cls = _ONNX_OPS_BY_NAME.get("ONNX" + op_name)
    if cls is None:
        return False

    class Expansion(ExpandTransformation):
        environments = []
        forward_impl = impl

        @classmethod
        def expansion(cls_, node, state, sdfg):
            node.validate(sdfg, state)
            if cls_.forward_impl.forward_can_be_applied(node, state, sdfg):
                result = cls_.forward_impl.forward(node, state, sdfg)
                if hasattr(cls_.forward_impl, "environments"):
                    cls_.environments.extend(cls_.forward_impl.environments)
                return result
            log.info('Falling back to onnxruntime expansion for library node "{}". '
                     'Reason: forward_can_be_applied returned False'.format(node.label))
            return expand_node(node, state, sdfg)

    Expansion.__name__ = f"{implementation_name}_{op_name}_Expansion"
    cls.register_implementation(implementation_name, Expansion)
    return True


# ------------------------------------------------------------------------------------
# class generation (onnx_op.py:494-694)

_ONNX_OPS_BY_NAME: typing.Dict[str, typing.Type[ONNXOp]] = {}


def _make_class(dace_schema: ONNXSchema):
    required_attrs = {name for name, attr in dace_schema.attributes.items() if attr.required}

    def __init__(self, name=None, *args, location=None, **op_attributes):
        if name is None:
            name = dace_schema.name
        LibraryNode.__init__(
            self, name, location=location,
            inputs={i.name for i in dace_schema.inputs if i.param_type == ONNXParameterType.Single},
            outputs={o.name for o in dace_schema.outputs if o.param_type == ONNXParameterType.Single})
        self.backward_implementation = None
        if len(args) > 0:
            raise TypeError("__init__() takes 1 positional arguments but {} were given".format(1 + len(args)))
        missing_arguments = required_attrs.difference(op_attributes)
        if len(missing_arguments) > 0:
            raise TypeError(get_missing_arguments_message("__init__()", sorted(missing_arguments),
                                                          "keyword-only argument"))
        unknown_attrs = set(op_attributes).difference(dace_schema.attributes)
        if len(unknown_attrs) > 0:
            raise TypeError("{}.__init__() got an unexpected keyword argument '{}'".format(
                dace_schema.name, sorted(unknown_attrs)[0]))
        # attributes are plain python attributes, None when unset (onnx_op.py:516-536)
        for attr_name, attr in dace_schema.attributes.items():
            default = attr.default_value
            setattr(self, attr_name, list(default) if isinstance(default, (list, tuple)) else default)
        for attr_name, value in op_attributes.items():
            setattr(self, attr_name, value)

    cls_name = "ONNX" + dace_schema.name
    attrs = {
        "__init__": __init__,
        "schema": dace_schema,
        "implementations": {},
        "default_implementation": None,
        "__doc__": "\n" + dace_schema.doc + "\n\n:Node Inputs: " +
                   ", ".join(p.name for p in dace_schema.inputs) + "\n:Node Outputs: " +
                   ", ".join(p.name for p in dace_schema.outputs) + "\n",
    }
    cls = type(cls_name, (ONNXOp, ), attrs)
    cls.register_implementation("onnxruntime", _make_ort_expansion())
    return cls_name, cls


for _schema in SCHEMAS:
    _name, _cls = _make_class(_schema)
    globals()[_name] = _cls
    _ONNX_OPS_BY_NAME[_name] = _cls
del _schema, _name, _cls


def has_onnx_node(name: str) -> bool:
    """Check if an ONNX operator is supported."""
    return ("ONNX" + name) in _ONNX_OPS_BY_NAME


def get_onnx_node(name: str) -> typing.Type[ONNXOp]:
    """Get the ONNX Operator node class for an operator by name."""
    return _ONNX_OPS_BY_NAME["ONNX" + name]

"""ONNX library nodes: one ``ONNX<Op>`` class per schema, with the reference's
construction, validation and implementation-binding behaviour
(``daceml/onnx/nodes/onnx_op.py:84-415`` ONNXOp and validate, ``:494-694`` class
generation and binding, ``:418-475`` the Python-frontend call form).
"""
import logging
import typing

from ...sdfg import SDFG, SDFGState, LibraryNode, MultiConnectorEdge
from ..schema import ONNXParameter, ONNXSchema, ONNXParameterType, SCHEMAS
from .node_utils import is_variadic_connector, parse_variadic_param

log = logging.getLogger(__name__)


def _missing_message(owner: str, names: typing.Sequence[str], kind: str) -> str:
    """Worded like Python's own report of missing arguments."""
    quoted = [f"'{n}'" for n in names]
    listing = quoted[0] if len(quoted) == 1 else ", ".join(quoted[:-1]) + ", and " + quoted[-1]
    return f"{owner} missing {len(names)} required {kind}{'' if len(names) == 1 else 's'}: {listing}"


def _is_private(connector: str) -> bool:
    # connectors with a leading underscore belong to one implementation (operands folded in by the
    # fusion pass); they are not schema parameters
    return connector.startswith("_")


class _Binding(typing.NamedTuple):
    """One edge of a node matched against its schema."""
    edge: MultiConnectorEdge
    is_input: bool
    connector: str
    parameter: typing.Optional[ONNXParameter]   # None: the schema has no parameter of that name
    index: typing.Optional[int]                 # position inside a variadic parameter
    position: typing.Tuple[int, int]            # sort key: (place in the schema, variadic index)


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

    # ---- edges matched against the schema ---------------------------------------------------
    def _bindings(self, state: SDFGState, inputs: bool) -> typing.List[_Binding]:
        """The node's (public) edges on one side, each resolved to its schema parameter, in schema order."""
        parameters = self.schema.inputs if inputs else self.schema.outputs
        place = {p.name: i for i, p in enumerate(parameters)}
        found = []
        for edge in (state.in_edges(self) if inputs else state.out_edges(self)):
            connector = edge.dst_conn if inputs else edge.src_conn
            if connector is None:
                raise ValueError("Edges to ONNX Ops must not have connector None")
            if _is_private(connector):
                continue
            base, index = parse_variadic_param(connector) if is_variadic_connector(connector) else (connector, None)
            parameter = parameters[place[base]] if base in place else None
            found.append(_Binding(edge, inputs, connector, parameter, index,
                                  (place.get(base, len(parameters)), index or 0)))
        found.sort(key=lambda b: b.position)
        return found

    def iter_inputs_in_onnx_order(self, state: SDFGState) -> typing.List[MultiConnectorEdge]:
        """Input edges ordered as the schema orders its parameters (``onnx_op.py:107-125``)."""
        return [b.edge for b in self._bindings(state, True) if b.parameter is not None]

    def iter_outputs_in_onnx_order(self, state: SDFGState) -> typing.List[MultiConnectorEdge]:
        return [b.edge for b in self._bindings(state, False) if b.parameter is not None]

    def iter_edges(self, state: SDFGState):
        """(edge, is_input) pairs, inputs first, each side in schema order (``onnx_op.py:127-189``)."""
        for inputs in (True, False):
            for b in self._bindings(state, inputs):
                if b.parameter is None:
                    raise ValueError(f"Found 0 connectors with name '{b.connector}', expected to find exactly one")
                yield b.edge, inputs

    # ---- validation: the contract of ``onnx_op.py:197-415`` ----------------------------------
    # every edge names a parameter of the schema and a connector of the node; every required parameter is
    # connected; the indices of a variadic parameter are 0..n-1, each once; all parameters that share a type
    # string carry one dtype, and it is one the schema allows; required attributes are set.
    def validate(self, sdfg: SDFG, state: SDFGState):
        sides = [(True, self._bindings(state, True)), (False, self._bindings(state, False))]
        for checker in (self._check_names, self._check_required, self._check_variadic_numbering):
            for inputs, bindings in sides:
                checker(inputs, bindings)
        self._check_dtypes(sdfg, [b for _, bindings in sides for b in bindings])
        unset = [name for name, attr in self.schema.attributes.items() if attr.required and getattr(self, name) is None]
        if unset:
            raise ValueError(f"Expected value for required attribute '{unset[0]}', got None")

    def _check_names(self, inputs: bool, bindings: typing.List[_Binding]):
        kind = "input" if inputs else "output"
        declared = self.in_connectors if inputs else self.out_connectors
        for b in bindings:
            if b.parameter is None:
                if b.index is None:
                    raise TypeError(f"Got an unexpected argument '{b.connector}'")
                raise ValueError(f"Got an unexpected variadic argument '{b.connector}'")
            if (b.index is not None) != (b.parameter.param_type == ONNXParameterType.Variadic):
                if b.index is not None:
                    raise ValueError(f"Got variadic argument '{b.connector}' for non-variadic parameter "
                                     f"'{b.parameter.name}'. Ensure that non-variadic args do not contain '__'")
                raise ValueError(f"Got an unexpected variadic argument '{b.connector}': variadic parameter "
                                 f"'{b.parameter.name}' is connected as '{b.parameter.name}__<index>'")
            if b.connector not in declared:
                raise ValueError(f"Memlet {b.edge.data} leading to nonexistent {kind} connector '{b.connector}'")

    def _check_required(self, inputs: bool, bindings: typing.List[_Binding]):
        connected = {b.parameter.name for b in bindings}
        missing = sorted(p.name for p in (self.schema.inputs if inputs else self.schema.outputs)
                         if p.param_type == ONNXParameterType.Single and p.name not in connected)
        if missing:
            raise ValueError(_missing_message(self.schema.name, missing, "input" if inputs else "output"))

    @staticmethod
    def _check_variadic_numbering(inputs: bool, bindings: typing.List[_Binding]):
        kind = "inputs" if inputs else "outputs"
        indices = [b.index for b in bindings if b.index is not None]   # at most one variadic parameter per side
        for number in indices:
            if indices.count(number) > 1:
                raise ValueError(f"Got two variadic {kind} with index {number}, expected at most one")
        for expected in range(len(indices)):
            if expected not in indices:
                raise ValueError(f"Since {len(indices)} variadic {kind} were passed, "
                                 f"expected variadic parameter with number {expected}")

    def _check_dtypes(self, sdfg: SDFG, bindings: typing.List[_Binding]):
        solved = {}   # type string -> dtype
        for b in bindings:
            kind = "input" if b.is_input else "output"
            dtype = sdfg.arrays[b.edge.data.data].dtype
            type_str = b.parameter.type_str
            allowed = self.schema.type_constraints[type_str].types
            if dtype != solved.get(type_str, dtype):
                raise ValueError(f"Could not solve type constraints; excepted type '{solved[type_str]}' for {kind} "
                                 f"'{b.parameter.name}', got type '{dtype}'")
            if dtype not in allowed:
                raise ValueError(f"Expected type in '{allowed}' for {kind} '{b.parameter.name}', got type '{dtype}'")
            solved[type_str] = dtype


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
            raise TypeError(_missing_message("__init__()", sorted(missing_arguments),
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

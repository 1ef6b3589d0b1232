"""``ONNXModel``: load an ONNX graph into an SDFG of ONNX library nodes and run it.

Follows ``daceml/onnx/onnx_importer.py``: inputs/outputs/value_infos become
arrays (``:155-166``), initializers become ``self.weights`` torch tensors passed
as ordinary arguments (``:177-178``, ``:424-442``), every graph node becomes an
``ONNX<Op>`` node whose connectors are named from the schema (``:182-299``), and
``__call__`` optimises, expands, compiles once and runs with positional arguments
bound to ``graph.input`` in order (``:444-572``), returning torch tensors when
any input is a torch tensor and numpy arrays otherwise (``:586-633``).

The model is a :class:`dace_onnx_amd.onnx.proto.ModelProto`, a path to a
``.onnx`` file, or serialized bytes. Everything executes on the GPU; weights are
uploaded once at construction.
"""
import collections
import logging
import re
import copy
import typing
from itertools import chain, repeat

import numpy as np
import torch

from .. import sdfg as dace
from ..sdfg import SDFG, SDFGState, AccessNode
from . import proto
from .proto import ModelProto, TensorProto
from .schema import ONNXParameterType
from .nodes.onnx_op import get_onnx_node, has_onnx_node
from .shape_inference import infer_shapes as _infer_shapes

log = logging.getLogger(__name__)


def clean_onnx_name(name: str) -> str:
    """Make an ONNX value name a valid array name (``daceml/onnx/converters.py:204-211``)."""
    if re.match("^[0-9]", name):
        name = f"ONNX_{name}"
    return name.replace(".", "DOT").replace(":", "COLON").replace("/", "SLASH").replace("-", "DASH")


def onnx_tensor_type_to_typeclass(elem_type: int) -> dace.typeclass:
    try:
        return dace.typeclass_of(proto.tensor_dtype_to_np_dtype(elem_type))
    except KeyError:
        raise ValueError(f"ONNX tensor element type {elem_type} is not supported")


class ONNXModel:
    """Loads an ONNX model into an SDFG and executes it on the MI355X.

    :Example:

        >>> model = dace_onnx_amd.onnx.proto.load("layer.onnx")     # doctest: +SKIP
        >>> dace_model = ONNXModel("layer", model)                    # doctest: +SKIP
        >>> out = dace_model(np.random.rand(8, 128, 768).astype(np.float32))  # doctest: +SKIP
    """

    def __init__(self,
                 name: str,
                 model: typing.Union[ModelProto, str, bytes],
                 infer_shapes: bool = True,
                 cuda: bool = True,
                 apply_strict: bool = False,
                 auto_optimize: bool = True,
                 fold_constants: bool = True,
                 parent_pytorch_module: typing.Optional[torch.nn.Module] = None,
                 fuse: bool = True,
                 use_hip_graph: bool = False,
                 save_transients: typing.Optional[typing.Dict[str, torch.Tensor]] = None,
                 storage=None,
                 auto_merge: bool = False):
        """
        :param name: the name for the SDFG.
        :param model: the model to import.
        :param infer_shapes: infer shapes of intermediate values; if ``False`` the model must carry
                             value_info for all of them.
        :param cuda: kept for signature compatibility; execution is always on the GPU.
        :param fold_constants: replace nodes whose inputs are all constants by their value
                               (``transformation/constant_folding.py``) before the graph is built.
        :param auto_optimize: apply the graph-level fusion pass before expanding (first call).
        :param parent_pytorch_module: when not None, weights whose names match parameters of this
                                      module are taken from it rather than from the ONNX graph.
        :param fuse: with ``auto_optimize``, fold bias/activation/residual/transposes into contractions.
        :param use_hip_graph: replay the launch sequence as one HIP graph from the second call on.
        :param storage: kept for signature compatibility (``onnx_importer.py:104``): parameters, inputs and
                        outputs always live in GPU global memory; anything else named here is an error.
        :param auto_merge: kept for signature compatibility (symbolic shape merging; shapes are static here).
        :param save_transients: if not None, every intermediate value of the graph is kept and stored in
                                this dict under its array name on each call (for debugging; as in the
                                reference, ``onnx_importer.py:454-478``, the intermediates stop being
                                transients, so nothing is fused across them).
        """
        if not isinstance(model, ModelProto):
            model = proto.load(model)
        if storage is not None and "GPU" not in str(storage):
            raise ValueError(f"storage {storage!r}: this runner keeps every array in GPU global memory")
        default_opset = 12
        for opset in model.opset_import:
            if opset.domain in ("", "ai.onnx"):
                default_opset = opset.version
                if opset.version not in (12, 17, 20):
                    log.warning(f"Expected the onnx model to be exported with opset 12, got {opset.version}. "
                                f"This model may fail to import as a result.")
        self.opset_version = default_opset  #: version of the default operator set the model imports
        self.do_auto_optimize = auto_optimize
        self.fuse = fuse
        self.use_hip_graph = use_hip_graph
        self.save_transients = save_transients
        if save_transients is not None and use_hip_graph:
            raise ValueError("save_transients allocates fresh tensors on every call: not with use_hip_graph")
        model = self._constants_to_initializers(model)
        if fold_constants:
            from ..transformation.constant_folding import fold_constants as _fold
            model = _fold(model)
        model = self._separate_passthrough_outputs(model)
        for node in model.graph.node:
            if not has_onnx_node(node.op_type):
                raise ValueError("Unsupported ONNX operator: '{}'".format(node.op_type))
        if infer_shapes:
            model = _infer_shapes(model)
        graph = model.graph

        self.sdfg: SDFG = SDFG(name)  #: the generated SDFG
        self.sdfg._parent_onnx_model = self
        self.cuda = True
        self.state: SDFGState = self.sdfg.add_state()  #: the state containing the model computation
        # Without a GPU the graph can still be imported, fused and expanded (weights stay
        # in host memory); compiling or calling it raises.
        self.device = torch.device("cuda:0" if torch.cuda.is_available() else "cpu")

        self.value_infos = {}
        self.inputs: typing.List[str] = []   #: the inputs to the model
        self.outputs: typing.List[str] = []  #: the outputs of the model
        initializer_names = {t.name for t in graph.initializer}

        for value, is_input in chain(zip(graph.input, repeat(True)), zip(graph.output, repeat(False))):
            if not value.name:
                raise ValueError("Got input or output without name")
            if is_input and value.name in initializer_names:
                # keep_initializers_as_inputs=True exports list every weight as an input
                self.value_infos[value.name] = value
                continue
            (self.inputs if is_input else self.outputs).append(value.name)
            self.value_infos[value.name] = value
            self._add_value_info(value, transient=False)
        for value in graph.value_info:
            if not value.name:
                raise ValueError("Got input or output without name")
            self.value_infos.setdefault(value.name, value)

        self.weights: typing.Dict[str, torch.Tensor] = {}  #: mapping from weight name to tensor
        for init in graph.initializer:
            self._add_constant_tensor(init, parent_pytorch_module)

        access_nodes = {}
        self._idx_to_node = []
        for i, node in enumerate(graph.node):
            if not has_onnx_node(node.op_type):
                raise ValueError("Unsupported ONNX operator: '{}'".format(node.op_type))
            op_attributes = {a.name: self._convert_attribute(a) for a in node.attribute}
            # Softmax / LogSoftmax without an axis attribute: the node classes carry the opset-11 default (1);
            # from opset 13 on the operator's default is the last axis
            if node.op_type in ("Softmax", "LogSoftmax") and "axis" not in op_attributes and self.opset_version >= 13:
                op_attributes["axis"] = -1
            node_name = clean_onnx_name(node.name) if node.name else node.op_type + "_" + str(i)
            op_node = get_onnx_node(node.op_type)(node_name, **op_attributes)
            self.state.add_node(op_node)
            self._idx_to_node.append(op_node)

            for param_idx, (vname, is_input) in chain(enumerate(zip(node.input, repeat(True))),
                                                      enumerate(zip(node.output, repeat(False)))):
                if vname == "":
                    continue  # omitted optional parameter
                if clean_onnx_name(vname) not in self.sdfg.arrays:
                    if vname not in self.value_infos:
                        raise ValueError("Could not find array with name '{}'".format(vname))
                    self._add_value_info(self.value_infos[vname], transient=True)
                if vname in access_nodes:
                    access = access_nodes[vname]
                else:
                    access = AccessNode(clean_onnx_name(vname))
                    self.state.add_node(access)
                    access_nodes[vname] = access
                params = op_node.schema.inputs if is_input else op_node.schema.outputs
                if param_idx >= len(params):
                    if not params or params[-1].param_type != ONNXParameterType.Variadic:
                        raise ValueError(
                            "Expected the last {i_or_o} parameter to be variadic, since the {i_or_o} with idx "
                            "{param_idx} has more parameters than the schema ({params_len})".format(
                                i_or_o="input" if is_input else "output", param_idx=param_idx,
                                params_len=len(params)))
                    conn_name = params[-1].name + "__" + str(param_idx - len(params) + 1)
                elif params[param_idx].param_type == ONNXParameterType.Variadic:
                    conn_name = params[param_idx].name + "__0"
                else:
                    conn_name = params[param_idx].name
                memlet = self.sdfg.make_array_memlet(clean_onnx_name(vname))
                if is_input:
                    op_node.add_in_connector(conn_name)
                    self.state.add_edge(access, None, op_node, conn_name, memlet)
                else:
                    op_node.add_out_connector(conn_name)
                    self.state.add_edge(op_node, conn_name, access, None, memlet)

        self._compiled = None
        self._expanded = False
        self._static_io = None

    # -- construction helpers ----------------------------------------------------------
    @staticmethod
    def _constants_to_initializers(model: ModelProto) -> ModelProto:
        """``Constant`` nodes become weights at import, as in the reference
        (``onnx_importer.py:193-229``, same checks and messages); here by turning each into an
        initializer named after its output before anything else looks at the graph. The
        caller's model is not modified."""
        if not any(n.op_type == "Constant" for n in model.graph.node):
            return model
        import copy
        model = copy.copy(model)
        model.graph = copy.copy(model.graph)
        possible_values = {"sparse_value", "value", "value_float", "value_floats", "value_int", "value_ints",
                           "value_string", "value_strings"}
        kept, extra = [], []
        for node in model.graph.node:
            if node.op_type != "Constant":
                kept.append(node)
                continue
            attrs = {a.name: a for a in node.attribute}
            if set(attrs).difference(possible_values):
                raise ValueError(f"Got unexpected attributes on Constant node {set(attrs).difference(possible_values)}")
            if len(attrs) != 1:
                raise ValueError("Expected Constant node to have exactly one of its attributes set")
            if len(node.input) != 0 or len(node.output) != 1:
                raise ValueError("Expected Constant node to have no inputs and exactly 1 output")
            (kind, attr), = attrs.items()
            if kind == "value":
                value = np.asarray(attr.value.array).reshape(attr.value.dims)
            elif kind == "value_float":
                value = np.asarray(attr.value, dtype=np.float32)
            elif kind == "value_floats":
                value = np.asarray(list(attr.value), dtype=np.float32)
            elif kind == "value_int":
                value = np.asarray(attr.value, dtype=np.int64)
            elif kind == "value_ints":
                value = np.asarray(list(attr.value), dtype=np.int64)
            else:
                raise ValueError(f"Constant node attribute '{kind}' is not supported")
            extra.append(proto.numpy_helper.from_array(value, name=node.output[0]))
        model.graph.node = kept
        model.graph.initializer = list(model.graph.initializer) + extra
        return model

    @staticmethod
    def _separate_passthrough_outputs(model: ModelProto) -> ModelProto:
        """A graph output that is a graph input or an initializer itself (legal ONNX; also what remains when
        constant folding consumes every node) gets an ``Identity`` node and a name of its own, so that the
        caller's output buffer and the input are two arrays. The caller's model is not modified."""
        graph = model.graph
        sources = {v.name for v in graph.input} | {t.name for t in graph.initializer}
        if not any(o.name in sources for o in graph.output):
            return model
        model = copy.copy(model)
        model.graph = graph = copy.copy(graph)
        taken = sources | {o for n in graph.node for o in n.output}
        graph.node, graph.output = list(graph.node), list(graph.output)
        for i, out in enumerate(graph.output):
            if out.name not in sources:
                continue
            new_name = out.name + "_output"
            while new_name in taken:
                new_name += "_"
            taken.add(new_name)
            graph.node.append(proto.helper.make_node("Identity", [out.name], [new_name], name="passthrough_" + new_name))
            renamed = copy.copy(out)
            renamed.name = new_name
            graph.output[i] = renamed
        return model

    @staticmethod
    def _convert_attribute(attr):
        v = attr.value
        if isinstance(v, TensorProto):
            return v.array
        if isinstance(v, bytes):
            return v.decode("utf-8")
        return list(v) if isinstance(v, (list, tuple)) else v

    def _add_value_info(self, value_info, transient: bool):
        name = value_info.name
        if value_info.shape is None or not all(isinstance(d, int) for d in value_info.shape):
            raise ValueError(f"value '{name}' has no static shape ({value_info.shape}); "
                             f"symbolic dimensions are not supported")
        self.sdfg.add_array(clean_onnx_name(name), value_info.shape,
                            onnx_tensor_type_to_typeclass(value_info.elem_type), transient=transient)

    def _add_constant_tensor(self, tensor: TensorProto, parent_pytorch_module):
        if not tensor.name:
            raise ValueError("Got tensor without name")
        name = clean_onnx_name(tensor.name)
        dtype = onnx_tensor_type_to_typeclass(tensor.data_type)
        if name not in self.sdfg.arrays:
            self.sdfg.add_array(name, tensor.dims, dtype, transient=False)
        else:
            desc = self.sdfg.arrays[name]
            if desc.dtype != dtype or tuple(desc.shape) != tuple(tensor.dims):
                raise ValueError(f"initializer '{tensor.name}' contradicts its value_info")
            desc.transient = False
        weight = None
        if parent_pytorch_module is not None:
            params = dict(parent_pytorch_module.named_parameters())
            params.update(dict(parent_pytorch_module.named_buffers()))
            if tensor.name in params:
                weight = params[tensor.name].detach()
        if weight is None:
            weight = torch.from_numpy(np.array(tensor.array, copy=True).reshape(tensor.dims))
        self.weights[tensor.name] = weight.to(self.device).contiguous()

    @property
    def clean_weights(self):
        return {clean_onnx_name(k): v for k, v in self.weights.items()}

    # -- execution ------------------------------------------------------------------------
    def auto_optimize(self):
        from ..util import utils
        utils.auto_optimize(self.sdfg, cuda=True, fuse=self.fuse)

    def expand(self):
        """Apply the graph-level fusion (if enabled) and expand every ONNX node to kernel
        calls; returns the SDFG. Needs no GPU."""
        if not self._expanded:
            if self.save_transients is not None:
                self._saved = [k for k, d in self.sdfg.arrays.items() if d.transient]
                for k in self._saved:
                    self.sdfg.arrays[k].transient = False
            if self.do_auto_optimize:
                self.auto_optimize()
            from ..util.utils import expand_onnx_nodes
            expand_onnx_nodes(self.sdfg)
            self._expanded = True
        return self.sdfg

    def expand_onnx_nodes(self):
        """Expand every ONNX node of the SDFG as it is (no fusion); the reference's method of the same
        name (``onnx_importer.py:574-575``). :meth:`expand` is the fusing variant ``__call__`` uses."""
        from ..util.utils import expand_onnx_nodes
        expand_onnx_nodes(self.sdfg)
        self._expanded = True

    def compile_and_init(self):
        if self._compiled is None:
            if self.device.type != "cuda":
                raise RuntimeError("ONNXModel executes on the MI355X only: no HIP device is visible")
            self.expand()
            self._compiled = self.sdfg.compile()
        return self._compiled

    def _call_args(self, args, kwargs):
        if len(args) > len(self.inputs):
            raise TypeError(f"expected at most {len(self.inputs)} positional arguments, got {len(args)}")
        inputs = dict(zip(self.inputs, args))
        for k, v in kwargs.items():
            if k not in self.inputs:
                raise TypeError(f"unknown input '{k}' (model inputs: {self.inputs})")
            if k in inputs:
                raise TypeError(f"got multiple values for input '{k}'")
            inputs[k] = v
        missing = [n for n in self.inputs if n not in inputs]
        if missing:
            raise TypeError(f"missing model inputs {missing}")
        return inputs

    def __call__(self, *args, **kwargs):
        """Execute the model.

        :param args: positional arguments; the i-th is the i-th graph input.
        :param kwargs: named arguments matching the ONNX input names.
        :return: the output (or a tuple of outputs): torch tensors on the GPU if any
                 input was a torch tensor, numpy arrays otherwise.
        """
        compiled = self.compile_and_init()
        inputs = self._call_args(args, kwargs)
        use_torch = any(isinstance(v, torch.Tensor) for v in inputs.values())
        call = {}
        for n, v in inputs.items():
            desc = self.sdfg.arrays[clean_onnx_name(n)]
            if isinstance(v, torch.Tensor):
                v = v.to(self.device)
                if not v.is_contiguous():
                    v = v.contiguous()
            else:
                v = torch.from_numpy(np.ascontiguousarray(np.asarray(v, dtype=desc.dtype.np_dtype))).to(self.device)
            call[clean_onnx_name(n)] = v
        outputs = collections.OrderedDict()
        if self.use_hip_graph:
            if self._static_io is None:
                # private input/output buffers: the graph is bound to their addresses
                s_in = {k: v.clone() for k, v in call.items()}
                s_out = {}
                for n in self.outputs:
                    desc = self.sdfg.arrays[clean_onnx_name(n)]
                    s_out[clean_onnx_name(n)] = torch.empty(desc.shape, dtype=desc.dtype.as_torch(), device=self.device)
                compiled(**s_in, **s_out, **self.clean_weights)  # eager run, binds the launch list
                compiled.capture_graph()
                self._static_io = (s_in, s_out)
            else:
                s_in, s_out = self._static_io
                for k, v in call.items():
                    s_in[k].copy_(v)
                compiled.replay()
            outputs = collections.OrderedDict((n, s_out[clean_onnx_name(n)].clone()) for n in self.outputs)
        else:
            for n in self.outputs:
                desc = self.sdfg.arrays[clean_onnx_name(n)]
                outputs[n] = torch.empty(desc.shape, dtype=desc.dtype.as_torch(), device=self.device)
            out_kwargs = {clean_onnx_name(n): t for n, t in outputs.items()}
            if self.save_transients is not None:
                for k in self._saved:
                    desc = self.sdfg.arrays[k]
                    out_kwargs[k] = self.save_transients[k] = torch.empty(desc.shape, dtype=desc.dtype.as_torch(),
                                                                          device=self.device)
            compiled(**call, **out_kwargs, **self.clean_weights)
        results = [t if use_torch else t.cpu().numpy() for t in outputs.values()]
        return results[0] if len(results) == 1 else tuple(results)


def create_output_array(inferred_symbols: typing.Dict[str, int], desc, use_torch: bool = False, zeros: bool = False):
    """The array for an output described by ``desc`` (``onnx_importer.py:586-633`` in the reference): a torch
    tensor on the GPU when ``use_torch``. Outputs live in device memory here, so ``use_torch=False`` is refused
    like the reference refuses a GPU descriptor without it. ``inferred_symbols`` is accepted for signature
    compatibility: shapes are static."""
    if not use_torch:
        raise ValueError("Got use_torch=False, but received a GPU descriptor")
    shape = [int(d) for d in desc.shape]
    make = torch.zeros if zeros else torch.empty
    device = torch.device("cuda:0" if torch.cuda.is_available() else "cpu")
    return make(shape if shape else [1], dtype=desc.dtype.as_torch(), device=device).reshape(shape)

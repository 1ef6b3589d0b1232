"""``DaceModule``: run a PyTorch ``nn.Module`` through the "mi355x" expansions.

Mirrors ``daceml/pytorch/module.py:28-322``: the wrapper turns the module into an
ONNX graph on its first call (shapes taken from the actual inputs, or from
``dummy_inputs``), imports it with ``ONNXModel`` (parameters are taken from the
module: ``parent_pytorch_module``, module.py:260-265), and from then on calls the
compiled graph on device tensors.

The reference obtains the ONNX graph from ``torch.onnx.export(opset_version=12,
do_constant_folding=False, keep_initializers_as_inputs=True)`` (module.py:238-256).
Two ways to the graph here (``exporter=``):

* ``"structural"``: the graph is written directly from the module structure, in the
  same opset-12 vocabulary the exporter uses -- ``nn.Linear`` becomes Gemm (2-D input)
  or MatMul + Add, ``nn.LayerNorm`` the nine-node ReduceMean ... Add chain, ``nn.GELU``
  the five-node Erf chain -- for the module types on the hot path: ``Sequential`` of
  Linear, Conv2d, ReLU, GELU, LayerNorm, Softmax, Flatten, Identity, Dropout
  (inference: identity), and ``transformers``' ``BertLayer`` (the module of
  tests/pytorch/test_bert_encoder.py:17). Anything else raises ``UnsupportedModule``.
* ``"torch"``: the reference's own call of the TorchScript exporter, any number of
  inputs, any module whose exported operators have an ``ONNX<Op>`` node here. The
  exporter's last step attaches onnxscript functions through the ``onnx`` package;
  when that package is absent the step is skipped for the duration of the call (the
  graphs concerned hold none).
* ``"auto"`` (default): structural where it applies, the exporter otherwise.

Inference only: ``backward=True`` is refused (the reference's autodiff is a separate
subsystem).
"""
import collections
import contextlib
import io
import logging
import math
import typing
import warnings
from functools import wraps

import numpy as np
import torch
import torch.nn as nn

from ..onnx.onnx_importer import ONNXModel
from ..onnx.proto import helper, numpy_helper, TensorProto, ModelProto


log = logging.getLogger(__name__)


class UnsupportedModule(NotImplementedError):
    """The module (or one of its children, or its configuration) has no ONNX form here."""


class _GraphBuilder:
    def __init__(self):
        self.nodes, self.inits, self.names = [], [], set()

    def fresh(self, hint):
        name, i = hint, 0
        while name in self.names:
            i += 1
            name = f"{hint}_{i}"
        self.names.add(name)
        return name

    def node(self, op, ins, hint, **attrs):
        out = self.fresh(hint)
        self.nodes.append(helper.make_node(op, list(ins), [out], name=f"{op}_{len(self.nodes)}", **attrs))
        return out

    def const(self, value, hint, dtype=np.float32):
        name = self.fresh(hint)
        self.inits.append(numpy_helper.from_array(np.asarray(value, dtype=dtype), name))
        return name

    def param(self, tensor, name):
        """Initializer named like the module parameter, so ONNXModel takes the live tensor from the module."""
        self.names.add(name)
        self.inits.append(numpy_helper.from_array(tensor.detach().cpu().numpy(), name))
        return name


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else tuple(int(e) for e in v)


def _linear(g, m, prefix, x, x_rank):
    if x_rank == 2:  # what the exporter emits for 2-D inputs: Gemm(transB=1) on the [out, in] weight
        ins = [x, g.param(m.weight, prefix + "weight")] + ([g.param(m.bias, prefix + "bias")] if m.bias is not None else [])
        return g.node("Gemm", ins, prefix + "out", alpha=1.0, beta=1.0, transB=1)
    # N-D inputs: MatMul with the transposed weight as a constant, then Add
    w_t = g.const(m.weight.detach().cpu().numpy().T.copy(), prefix + "weight_t")
    y = g.node("MatMul", [x, w_t], prefix + "mm")
    return g.node("Add", [y, g.param(m.bias, prefix + "bias")], prefix + "out") if m.bias is not None else y


def _layer_norm(g, m, prefix, x, x_rank):
    if len(m.normalized_shape) != 1 or not m.elementwise_affine:
        raise UnsupportedModule("LayerNorm over one trailing dimension with affine parameters only")
    mean = g.node("ReduceMean", [x], prefix + "mean", axes=[-1], keepdims=1)
    centred = g.node("Sub", [x, mean], prefix + "centred")
    sq = g.node("Pow", [centred, g.const(2.0, prefix + "two")], prefix + "sq")
    var = g.node("ReduceMean", [sq], prefix + "var", axes=[-1], keepdims=1)
    std = g.node("Sqrt", [g.node("Add", [var, g.const(m.eps, prefix + "eps")], prefix + "var_eps")], prefix + "std")
    normed = g.node("Div", [centred, std], prefix + "normed")
    scaled = g.node("Mul", [normed, g.param(m.weight, prefix + "weight")], prefix + "scaled")
    return g.node("Add", [scaled, g.param(m.bias, prefix + "bias")], prefix + "out") if m.bias is not None else scaled


def _gelu(g, prefix, x):
    t = g.node("Div", [x, g.const(math.sqrt(2.0), prefix + "sqrt2")], prefix + "scaled")
    t = g.node("Add", [g.node("Erf", [t], prefix + "erf"), g.const(1.0, prefix + "one")], prefix + "erf1")
    return g.node("Mul", [g.node("Mul", [x, t], prefix + "xerf"), g.const(0.5, prefix + "half")], prefix + "out")


def _bert_layer(g, m, prefix, x, shape):
    att, so = m.attention.self, m.attention.output
    if len(shape) != 3:
        raise UnsupportedModule("BertLayer expects [batch, seq, hidden] input")
    batch, seq, hidden = shape
    heads = int(att.num_attention_heads)
    d = hidden // heads
    if getattr(m, "is_decoder", False) or getattr(m, "add_cross_attention", False):
        raise UnsupportedModule("decoder / cross-attention BertLayer")
    act = m.intermediate.intermediate_act_fn
    if not (isinstance(act, nn.GELU) or type(act).__name__ in ("GELUActivation", "GELU") or act is torch.nn.functional.gelu):
        raise UnsupportedModule(f"BertLayer activation {act!r}: only exact gelu")
    split = g.const([batch, seq, heads, d], prefix + "split_shape", np.int64)
    merge = g.const([batch, seq, hidden], prefix + "merge_shape", np.int64)

    def heads_of(lin, tag):
        y = _linear(g, lin, f"{prefix}attention.self.{tag}.", x, 3)
        return g.node("Transpose", [g.node("Reshape", [y, split], f"{prefix}{tag}_4d")], f"{prefix}{tag}_heads", perm=[0, 2, 1, 3])

    q, k, v = heads_of(att.query, "query"), heads_of(att.key, "key"), heads_of(att.value, "value")
    kt = g.node("Transpose", [k], prefix + "key_t", perm=[0, 1, 3, 2])
    scores = g.node("Div", [g.node("MatMul", [q, kt], prefix + "scores_raw"), g.const(math.sqrt(d), prefix + "sqrt_d")],
                    prefix + "scores")
    probs = g.node("Softmax", [scores], prefix + "probs", axis=3)
    ctx = g.node("Transpose", [g.node("MatMul", [probs, v], prefix + "ctx_heads")], prefix + "ctx_t", perm=[0, 2, 1, 3])
    ctx = g.node("Reshape", [ctx, merge], prefix + "ctx")
    attn = _linear(g, so.dense, prefix + "attention.output.dense.", ctx, 3)
    h1 = _layer_norm(g, so.LayerNorm, prefix + "attention.output.LayerNorm.", g.node("Add", [attn, x], prefix + "attn_res"), 3)
    inter = _gelu(g, prefix + "intermediate.gelu.", _linear(g, m.intermediate.dense, prefix + "intermediate.dense.", h1, 3))
    out = _linear(g, m.output.dense, prefix + "output.dense.", inter, 3)
    return _layer_norm(g, m.output.LayerNorm, prefix + "output.LayerNorm.", g.node("Add", [out, h1], prefix + "ffn_res"), 3), shape


def _convert(g, m, prefix, x, shape):
    """Append the nodes of ``m`` applied to value ``x`` of ``shape``; returns (output value, output shape)."""
    shape = list(shape)
    if isinstance(m, nn.Sequential):
        for name, child in m.named_children():
            x, shape = _convert(g, child, f"{prefix}{name}.", x, shape)
        return x, shape
    if isinstance(m, (nn.Identity, nn.Dropout)):
        return x, shape
    if isinstance(m, nn.Linear):
        return _linear(g, m, prefix, x, len(shape)), shape[:-1] + [m.out_features]
    if isinstance(m, nn.Conv2d):
        if m.groups != 1 or m.padding_mode != "zeros" or isinstance(m.padding, str) or len(shape) != 4:
            raise UnsupportedModule("Conv2d: group 1, zero padding given as numbers, NCHW input")
        (ph, pw), (sh, sw), (dh, dw), (kh, kw) = _pair(m.padding), _pair(m.stride), _pair(m.dilation), _pair(m.kernel_size)
        ins = [x, g.param(m.weight, prefix + "weight")] + ([g.param(m.bias, prefix + "bias")] if m.bias is not None else [])
        y = g.node("Conv", ins, prefix + "out", kernel_shape=[kh, kw], pads=[ph, pw, ph, pw], strides=[sh, sw],
                   dilations=[dh, dw], group=1)
        oh = (shape[2] + 2 * ph - dh * (kh - 1) - 1) // sh + 1
        ow = (shape[3] + 2 * pw - dw * (kw - 1) - 1) // sw + 1
        return y, [shape[0], m.out_channels, oh, ow]
    if isinstance(m, nn.BatchNorm2d):
        if m.training or not m.track_running_stats or not m.affine or len(shape) != 4:
            raise UnsupportedModule("BatchNorm2d: eval() mode with running statistics and affine parameters, NCHW input")
        ins = [x, g.param(m.weight, prefix + "weight"), g.param(m.bias, prefix + "bias"),
               g.param(m.running_mean, prefix + "running_mean"), g.param(m.running_var, prefix + "running_var")]
        return g.node("BatchNormalization", ins, prefix + "out", epsilon=float(m.eps), momentum=float(1.0 - (m.momentum or 0.1))), shape
    if isinstance(m, nn.MaxPool2d):
        if m.ceil_mode or m.return_indices or len(shape) != 4:
            raise UnsupportedModule("MaxPool2d: floor output size, no indices, NCHW input")
        (kh, kw), (ph, pw), (dh, dw) = _pair(m.kernel_size), _pair(m.padding), _pair(m.dilation)
        sh, sw = _pair(m.stride if m.stride is not None else m.kernel_size)
        y = g.node("MaxPool", [x], prefix + "out", kernel_shape=[kh, kw], pads=[ph, pw, ph, pw], strides=[sh, sw], dilations=[dh, dw])
        oh = (shape[2] + 2 * ph - dh * (kh - 1) - 1) // sh + 1
        ow = (shape[3] + 2 * pw - dw * (kw - 1) - 1) // sw + 1
        return y, [shape[0], shape[1], oh, ow]
    if isinstance(m, nn.AdaptiveAvgPool2d):
        if _pair(m.output_size) != (1, 1) or len(shape) != 4:
            raise UnsupportedModule("AdaptiveAvgPool2d(1) only (GlobalAveragePool)")
        return g.node("GlobalAveragePool", [x], prefix + "out"), [shape[0], shape[1], 1, 1]
    if isinstance(m, nn.ReLU):
        return g.node("Relu", [x], prefix + "out"), shape
    if isinstance(m, nn.GELU):
        if m.approximate != "none":
            raise UnsupportedModule("GELU(approximate='tanh')")
        return _gelu(g, prefix, x), shape
    if isinstance(m, nn.LayerNorm):
        return _layer_norm(g, m, prefix, x, len(shape)), shape
    if isinstance(m, nn.Softmax):
        if m.dim is None:
            raise UnsupportedModule("Softmax without dim")
        return g.node("Softmax", [x], prefix + "out", axis=int(m.dim) % len(shape)), shape
    if isinstance(m, nn.Flatten):
        if m.start_dim != 1 or m.end_dim not in (-1, len(shape) - 1):
            raise UnsupportedModule("Flatten(start_dim=1, end_dim=-1) only")
        return g.node("Flatten", [x], prefix + "out", axis=1), [shape[0], int(np.prod(shape[1:]))]
    if type(m).__name__ == "BertLayer":
        return _bert_layer(g, m, prefix, x, shape)
    raise UnsupportedModule(f"no ONNX form for {type(m).__name__}")


def module_to_onnx(module: nn.Module, dummy_inputs: typing.Sequence[torch.Tensor], name: str = "module") -> ModelProto:
    """ONNX graph (opset-12 vocabulary) of ``module`` for one float32 input of the given shape."""
    if len(dummy_inputs) != 1:
        raise UnsupportedModule("modules with exactly one tensor input")
    x = dummy_inputs[0]
    if x.dtype != torch.float32:
        raise UnsupportedModule(f"float32 inputs only, got {x.dtype}")
    g = _GraphBuilder()
    g.names.add("input")
    out, _ = _convert(g, module, "", "input", list(x.shape))
    if out == "input":
        out = g.node("Identity", ["input"], "output")
    graph = helper.make_graph(g.nodes, name, [helper.make_tensor_value_info("input", TensorProto.FLOAT, list(x.shape))],
                              [helper.make_tensor_value_info(out, TensorProto.FLOAT, None)], initializer=g.inits)
    return helper.make_model(graph, opset_imports=[helper.make_opsetid("", 12)])


@contextlib.contextmanager
def _exporter_without_onnx_package():
    """The TorchScript exporter serializes the graph itself; only its final ``_add_onnxscript_fn`` step
    imports ``onnx``. Without that package, replace the step by the identity while exporting."""
    try:
        import onnx  # noqa: F401
        yield
        return
    except ImportError:
        pass
    from torch.onnx._internal.torchscript_exporter import onnx_proto_utils
    saved = onnx_proto_utils._add_onnxscript_fn
    onnx_proto_utils._add_onnxscript_fn = lambda model_bytes, custom_opsets: model_bytes
    try:
        yield
    finally:
        onnx_proto_utils._add_onnxscript_fn = saved


def export_with_torch(module: nn.Module, dummy_inputs: typing.Sequence[torch.Tensor]) -> bytes:
    """``torch.onnx.export`` with the reference's arguments (daceml/pytorch/module.py:238-256): opset 12, no
    constant folding (folded weights lose the names that tie them to the module's parameters), initializers
    kept as inputs. Returns the serialized model."""
    # tracing runs the module: inputs go where its parameters are (only their shapes and types matter)
    where = next((p.device for p in module.parameters()), torch.device("cpu"))
    dummy_inputs = tuple(torch.zeros(t.shape, dtype=t.dtype, device=where) for t in dummy_inputs)
    buf = io.BytesIO()
    with _exporter_without_onnx_package(), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        torch.onnx.export(module, dummy_inputs, buf, opset_version=12, dynamo=False, do_constant_folding=False,
                          keep_initializers_as_inputs=True)
    return buf.getvalue()


class DaceModule(nn.Module):
    """A wrapper that runs a PyTorch ``nn.Module`` on the "mi355x" expansions.

    :param module: the model to wrap.
    :param dummy_inputs: a tuple of tensors whose shapes fix the graph; if None, the first call's inputs do.
    :param cuda: kept for signature compatibility: execution is always on the GPU.
    :param training: must be False (the graph is the inference graph).
    :param backward: must be False.
    :param auto_optimize: apply the graph-level fusion pass (registered as the post-ONNX hook "auto_optimize").
    :param use_hip_graph: replay the launch sequence as one HIP graph from the second call on (inputs are copied
                          into the graph's buffers; not in the reference, whose launches go through DaCe's streams).
    :param debug_transients: every intermediate value becomes an additional output of the module (a post-ONNX
                             hook placed before the optimisation, so nothing is fused across them).
    :param sdfg_name: the name to give to the SDFG (defaults to the module's class name).
    :param exporter: "auto", "structural" or "torch": how the ONNX graph is obtained (see the module docstring).

    Parameters are read from ``module`` when the graph is built (first call): derived copies (k-contiguous,
    concatenated weights) are made then, so call :meth:`reset_sdfg` after changing parameters.
    """

    def __init__(self, module: nn.Module, dummy_inputs: typing.Optional[typing.Tuple[torch.Tensor]] = None,
                 cuda: typing.Optional[bool] = None, training: bool = False, backward=False, apply_strict: bool = True,
                 auto_optimize: bool = True, debug_transients: bool = False, sdfg_name: typing.Optional[str] = None,
                 exporter: str = "auto", use_hip_graph: bool = False):
        super().__init__()
        self.use_hip_graph = use_hip_graph
        if exporter not in ("auto", "structural", "torch"):
            raise ValueError(f"exporter must be 'auto', 'structural' or 'torch', got {exporter!r}")
        self.exporter = exporter
        if backward or training:
            raise NotImplementedError("DaceModule here is inference only (backward=False, training=False)")
        self.model = module
        self.dace_model: typing.Optional[ONNXModel] = None
        self.onnx_model: typing.Optional[ModelProto] = None
        self.sdfg = None
        self.use_cuda = True
        self.sdfg_name = sdfg_name or type(module).__name__
        self.auto_optimize = auto_optimize
        self.debug_transients = debug_transients
        self.function = None
        #: hooks executed after the ONNX graph is imported to an SDFG, each called with this module
        self.post_onnx_hooks: "collections.OrderedDict[str, typing.Callable]" = collections.OrderedDict()
        #: hooks executed after the SDFG is compiled, each called with the compiled SDFG
        self.post_compile_hooks: "collections.OrderedDict[str, typing.Callable]" = collections.OrderedDict()

        # the reference's own use of its hooks (daceml/pytorch/module.py:98-146): the debugging option first,
        # the optimisation pass last, so that user hooks appended later run on the optimised graph
        if debug_transients:
            def transients_outputs(dace_module):
                model = dace_module.dace_model
                for name, desc in model.sdfg.arrays.items():
                    if desc.transient:
                        desc.transient = False
                        model.outputs.append(name)
            self.prepend_post_onnx_hook("make_transients_outputs", transients_outputs)
        if auto_optimize:
            def auto_optimize_hook(dace_module):
                from ..util import utils
                utils.auto_optimize(dace_module.dace_model.sdfg, cuda=True)
                dace_module.dace_model._expanded = True
            self.append_post_onnx_hook("auto_optimize", auto_optimize_hook)
        if dummy_inputs is not None:
            self.function = self._initialize_sdfg(dummy_inputs)

    def reset_sdfg(self):
        """Drop the compiled graph; the next call rebuilds it from the module's current parameters."""
        self.function = None
        self.dace_model = self.onnx_model = self.sdfg = None

    @staticmethod
    def _unique(existing, name):
        candidate, i = name, 0
        while candidate in existing:
            i += 1
            candidate = f"{name}_{i}"
        return candidate

    def _add_hook(self, hooks, name, func, first):
        if self.function is not None:
            log.warning("Added a hook after the model was already initialized. This hook will not be executed "
                        "until reset_sdfg() is called.")
        name = self._unique(hooks, name)
        hooks[name] = func
        if first:
            hooks.move_to_end(name, last=False)

    def prepend_post_onnx_hook(self, name: str, func: typing.Callable[["DaceModule"], None]):
        self._add_hook(self.post_onnx_hooks, name, func, first=True)

    def append_post_onnx_hook(self, name: str, func: typing.Callable[["DaceModule"], None]):
        self._add_hook(self.post_onnx_hooks, name, func, first=False)

    def prepend_post_compile_hook(self, name: str, func: typing.Callable):
        self._add_hook(self.post_compile_hooks, name, func, first=True)

    def append_post_compile_hook(self, name: str, func: typing.Callable):
        self._add_hook(self.post_compile_hooks, name, func, first=False)

    def _initialize_sdfg(self, dummy_inputs):
        was_training = self.model.training
        self.model.eval()
        try:
            self.onnx_model = None
            if self.exporter != "torch":
                try:
                    self.onnx_model = module_to_onnx(self.model, dummy_inputs, name=self.sdfg_name)
                except UnsupportedModule:
                    if self.exporter == "structural":
                        raise
            if self.onnx_model is None:
                from ..onnx import proto
                self.onnx_model = proto.parse_model(export_with_torch(self.model, dummy_inputs))
        finally:
            self.model.train(was_training)
        # optimisation is a hook of this module, not of the ONNXModel (which would apply it on its first call)
        self.dace_model = ONNXModel(self.sdfg_name, self.onnx_model, cuda=True, parent_pytorch_module=self.model,
                                    auto_optimize=False, use_hip_graph=self.use_hip_graph)
        self.sdfg = self.dace_model.sdfg
        for hook in self.post_onnx_hooks.values():
            hook(self)
        self._input_shapes = tuple(tuple(t.shape) for t in dummy_inputs)
        state = {"compiled": None}

        def forward(*args):
            if tuple(tuple(a.shape) for a in args) != self._input_shapes:
                raise TypeError(f"{self.sdfg_name} was built for inputs of shapes {self._input_shapes}")
            if state["compiled"] is None:     # needs the GPU: done on the first call, not at construction
                state["compiled"] = self.dace_model.compile_and_init()
                for hook in self.post_compile_hooks.values():
                    hook(state["compiled"])
            return self.dace_model(*args)

        return forward

    def forward(self, *actual_inputs):
        """Execute the forward pass on the GPU; torch tensors in, torch tensor on the GPU out."""
        if self.function is None:
            self.function = self._initialize_sdfg(actual_inputs)
        return self.function(*actual_inputs)


def dace_module(moduleclass=None, **wrapper_kwargs):
    """Decorator for an ``nn.Module`` class: instances are wrapped in :class:`DaceModule` on construction
    (daceml/pytorch/module.py:324-372). Usable bare (``@dace_module``) or with DaceModule's keyword arguments."""
    def decorate(cls):
        @wraps(cls)
        def _create(*args, **kwargs):
            return DaceModule(cls(*args, **kwargs), **wrapper_kwargs)
        return _create
    return decorate(moduleclass) if moduleclass is not None else decorate

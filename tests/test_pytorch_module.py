"""DaceModule: nn.Module -> ONNX graph -> "mi355x" expansions (the reference's tests/pytorch/
test_bert_encoder.py, test_module_conv-style checks). Host-side structure without a GPU, results
against the module itself evaluated in float64 on the CPU with one."""
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn

from dace_onnx_amd import sdfg as dace
from dace_onnx_amd.pytorch import DaceModule, dace_module, module_to_onnx, UnsupportedModule
from dace_onnx_amd.testing.utils import torch_tensors_close
from conftest import rel_err, FP32_REL_TOL


def _bert_layer(hidden=768, heads=12, ffn=3072):
    from transformers import BertConfig
    from transformers.models.bert.modeling_bert import BertLayer
    cfg = BertConfig(hidden_size=hidden, num_attention_heads=heads, intermediate_size=ffn, hidden_act="gelu",
                     layer_norm_eps=1e-12, attention_probs_dropout_prob=0.0, hidden_dropout_prob=0.0)
    cfg._attn_implementation = "eager"
    torch.manual_seed(0)
    return BertLayer(cfg).eval()


def _functions(dm):
    return [n.function for n, _ in dm.dace_model.expand().all_nodes_recursive() if isinstance(n, dace.KernelCall)]


def test_sequential_is_written_in_the_exporters_vocabulary():
    m = nn.Sequential(nn.Linear(8, 16), nn.GELU(), nn.LayerNorm(16), nn.Dropout(0.1), nn.Linear(16, 4), nn.Softmax(dim=-1))
    ops = [n.op_type for n in module_to_onnx(m, (torch.randn(5, 8), )).graph.node]
    assert ops == ["Gemm", "Div", "Erf", "Add", "Mul", "Mul", "ReduceMean", "Sub", "Pow", "ReduceMean", "Add", "Sqrt",
                   "Div", "Mul", "Add", "Gemm", "Softmax"]
    names = {i.name for i in module_to_onnx(m, (torch.randn(5, 8), )).graph.initializer}
    assert {"0.weight", "0.bias", "2.weight", "2.bias", "4.weight", "4.bias"} <= names   # parameter names survive
    dm = DaceModule(m, dummy_inputs=(torch.randn(5, 8), ))
    assert sorted(_functions(dm)) == ["mi355x_gemm_f32", "mi355x_gemm_f32", "mi355x_layernorm_f32", "mi355x_softmax_f32"]


def test_transformers_bert_layer_becomes_seven_launches():
    dm = DaceModule(_bert_layer(), dummy_inputs=(torch.randn(2, 128, 768), ))
    fns = _functions(dm)
    assert sorted(fns) == ["mi355x_attention_f32"] + ["mi355x_gemm_f32"] * 4 + ["mi355x_layernorm_f32"] * 2


def test_unsupported_modules_and_modes_are_refused():
    with pytest.raises(UnsupportedModule, match="LSTM"):
        module_to_onnx(nn.LSTM(4, 4), (torch.randn(2, 3, 4), ))
    with pytest.raises(UnsupportedModule, match="tanh"):
        module_to_onnx(nn.GELU(approximate="tanh"), (torch.randn(2, 4), ))
    with pytest.raises(UnsupportedModule, match="group"):
        module_to_onnx(nn.Conv2d(4, 4, 3, groups=2), (torch.randn(1, 4, 8, 8), ))
    with pytest.raises(NotImplementedError, match="inference only"):
        DaceModule(nn.ReLU(), backward=True)


@pytest.mark.gpu
def test_bert_encoder_layer_module():
    # the reference's test_bert_encoder.py: DaceModule(BertLayer) against the PyTorch module
    layer = _bert_layer()
    x = torch.randn(8, 128, 768)
    with torch.no_grad():
        ref = layer.double()(x.double())
        ref = ref[0] if isinstance(ref, (tuple, list)) else ref
    dace_layer = DaceModule(layer.float())
    got = dace_layer(x.cuda())
    assert got.is_cuda and got.dtype == torch.float32
    assert rel_err(ref.numpy(), got.cpu().numpy()) < FP32_REL_TOL
    torch_tensors_close("output", ref.float(), got.cpu(), rtol=1e-4, atol=1e-4)
    assert dace_layer.dace_model.compile_and_init().num_launches == 7
    with pytest.raises(TypeError, match="was built for"):
        dace_layer(torch.randn(4, 128, 768).cuda())


@pytest.mark.gpu
def test_conv_relu_linear_module_and_decorator():
    @dace_module
    class Net(nn.Sequential):
        def __init__(self):
            super().__init__(nn.Conv2d(32, 48, 3, padding=1), nn.ReLU(), nn.Conv2d(48, 16, 1, stride=2, bias=False),
                             nn.Flatten(), nn.Linear(16 * 6 * 6, 40), nn.ReLU(), nn.Linear(40, 10), nn.Softmax(dim=1))

    torch.manual_seed(1)
    net = Net()
    assert isinstance(net, DaceModule)
    x = torch.randn(6, 32, 12, 12)
    with torch.no_grad():
        ref = copy.deepcopy(net.model).double()(x.double())
    got = net(x.cuda())
    assert rel_err(ref.numpy(), got.cpu().numpy()) < FP32_REL_TOL
    # parameters changed after the graph was built: rebuilt on request
    with torch.no_grad():
        net.model[6].bias.add_(1.0)
        ref2 = copy.deepcopy(net.model).double()(x.double())
    net.reset_sdfg()
    assert rel_err(ref2.numpy(), net(x.cuda()).cpu().numpy()) < FP32_REL_TOL


def _small_resnet_stem():
    """Conv, BatchNorm, ReLU, MaxPool, Conv (no bias), BatchNorm, ReLU, global average pooling, Linear: the
    layer types of a ResNet around its 3 x 3 convolutions, in eval() mode with non-trivial statistics."""
    torch.manual_seed(5)
    net = nn.Sequential(nn.Conv2d(3, 8, 3, padding=1), nn.BatchNorm2d(8), nn.ReLU(), nn.MaxPool2d(3, 2, 1),
                        nn.Conv2d(8, 16, 3, padding=1, bias=False), nn.BatchNorm2d(16, eps=1e-3), nn.ReLU(),
                        nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(16, 10)).eval()
    with torch.no_grad():
        for m in net:
            if isinstance(m, nn.BatchNorm2d):
                m.running_mean.normal_()
                m.running_var.uniform_(0.5, 2.0)
                m.weight.normal_()
                m.bias.normal_()
    return net


@pytest.mark.parametrize("exporter", ["structural", "torch"])
def test_conv_batchnorm_pool_network_launch_list(exporter):
    net = _small_resnet_stem()
    dummy = (torch.randn(2, 3, 16, 16), )
    dm = DaceModule(net, dummy_inputs=dummy, exporter=exporter)
    # both BatchNormalizations folded into their convolutions, both ReLUs into the convolutions' epilogues
    assert _functions(dm) == ["mi355x_conv2d_f32", "mi355x_maxpool2d_f32", "mi355x_conv2d_f32", "mi355x_reduce_mean_f32",
                              "mi355x_gemm_f32"]
    plain = DaceModule(net, dummy_inputs=dummy, exporter=exporter, auto_optimize=False)
    assert sorted(_functions(plain)) == sorted(["mi355x_conv2d_f32", "mi355x_batchnorm_f32", "mi355x_eltwise_f32"] * 2 +
                                               ["mi355x_maxpool2d_f32", "mi355x_reduce_mean_f32", "mi355x_gemm_f32"])
    with pytest.raises(UnsupportedModule, match="eval"):
        module_to_onnx(copy.deepcopy(net).train(), dummy)


@pytest.mark.gpu
@pytest.mark.parametrize("exporter", ["structural", "torch"])
def test_conv_batchnorm_pool_network_results(exporter):
    net = _small_resnet_stem()
    x = torch.randn(4, 3, 16, 16)
    with torch.no_grad():
        ref = copy.deepcopy(net).double()(x.double())
    got = DaceModule(net, exporter=exporter)(x.cuda())
    assert rel_err(ref.numpy(), got.cpu().numpy()) < FP32_REL_TOL
    plain = DaceModule(net, exporter=exporter, auto_optimize=False)
    assert rel_err(ref.numpy(), plain(x.cuda()).cpu().numpy()) < FP32_REL_TOL


class _LeNet(nn.Module):
    """The network of the reference's tests/pytorch/test_lenet.py:14-34."""
    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(1, 6, (3, 3))
        self.conv2 = nn.Conv2d(6, 16, (3, 3))
        self.fc1 = nn.Linear(16 * 6 * 6, 120)
        self.fc2 = nn.Linear(120, 84)
        self.fc3 = nn.Linear(84, 10)

    def forward(self, x):
        F = torch.nn.functional
        x = F.max_pool2d(F.relu(self.conv1(x)), 2)
        x = F.max_pool2d(F.relu(self.conv2(x)), 2)
        x = x.view(-1, 16 * 6 * 6)
        x = F.relu(self.fc1(x))
        x = F.relu(self.fc2(x))
        x = self.fc3(x)
        return F.log_softmax(x, dim=1)


def test_lenet_launch_list():
    dm = DaceModule(_LeNet(), dummy_inputs=(torch.rand(8, 1, 32, 32), ))
    assert [n.op_type for n in dm.onnx_model.graph.node] == ["Conv", "Relu", "MaxPool", "Conv", "Relu", "MaxPool", "Constant",
                                                             "Reshape", "Gemm", "Relu", "Gemm", "Relu", "Gemm", "LogSoftmax"]
    # every Relu rides in the epilogue of the Conv / Gemm before it, the view is free
    assert _functions(dm) == ["mi355x_conv2d_f32", "mi355x_maxpool2d_f32", "mi355x_conv2d_f32", "mi355x_maxpool2d_f32",
                              "mi355x_gemm_f32", "mi355x_gemm_f32", "mi355x_gemm_f32", "mi355x_log_softmax_f32"]


@pytest.mark.gpu
def test_lenet_hip_graph_replay(sdfg_name):
    torch.manual_seed(10)
    net = _LeNet()
    dace_net = DaceModule(copy.deepcopy(net), sdfg_name=sdfg_name, use_hip_graph=True)
    for i in range(4):        # the first call runs eagerly and captures, the others replay
        input = torch.rand(8, 1, 32, 32)
        torch_tensors_close(f"output_{i}", net(input), dace_net(input.cuda()).cpu())
        torch.cuda.synchronize()


@pytest.mark.gpu
@pytest.mark.parametrize("use_hip_graph", [False, True])
def test_module_whose_output_is_a_view_eager_and_as_hip_graph(sdfg_name, use_hip_graph):
    """A network that ends in Flatten: the graph output is a Reshape of the last kernel's result. The producer
    writes straight into the output buffer (no copy, nothing that a HIP graph could not hold); several calls,
    each checked, with the caller keeping earlier results alive (so every eager call sees new output buffers)."""
    torch.manual_seed(12)
    net = nn.Sequential(nn.Conv2d(3, 8, 3, padding=1), nn.ReLU(), nn.Flatten()).eval()
    dace_net = DaceModule(copy.deepcopy(net), sdfg_name=sdfg_name, use_hip_graph=use_hip_graph)
    kept = []
    for i in range(4):
        input = torch.rand(2, 3, 6, 6)
        out = dace_net(input.cuda())
        kept.append((net(input), out))
        torch.cuda.synchronize()
    for i, (want, got) in enumerate(kept):
        torch_tensors_close(f"output_{i}", want, got.cpu())
    compiled = dace_net.dace_model.compile_and_init()
    assert compiled.num_launches == 1 and not any(item[0] == "copy" for item in compiled._launch_list)
    assert len(compiled._transient_tensors) <= 1   # allocated once, however many times the outputs changed


@pytest.mark.gpu
def test_lenet(sdfg_name):
    # tests/pytorch/test_lenet.py:37-57
    torch.manual_seed(7)
    input = torch.rand(8, 1, 32, 32, dtype=torch.float32)
    net = _LeNet()
    dace_net = _LeNet()
    dace_net.load_state_dict(net.state_dict())
    dace_net = DaceModule(dace_net, sdfg_name=sdfg_name)
    torch_output = net(torch.clone(input))
    dace_output = dace_net(torch.clone(input).cuda())
    torch_tensors_close("output", torch_output, dace_output.cpu())


class _ReshapeModel(nn.Module):
    def __init__(self, new_shape):
        super().__init__()
        self.new_shape = new_shape

    def forward(self, x):
        return x.reshape(self.new_shape)


@pytest.mark.gpu
def test_reshape_module_global_avg_pool_and_batchnorm(sdfg_name):
    # tests/pytorch/test_reshape.py:19-34
    x = torch.rand([25])
    dace_model = DaceModule(_ReshapeModel([5, 5]), auto_optimize=False, dummy_inputs=(x, ), sdfg_name=sdfg_name)
    torch_tensors_close("output", x.reshape(5, 5), dace_model(x.cuda()).cpu())
    # tests/pytorch/test_img_op_implementations.py:36-49
    inputs = torch.rand(1, 64, 60, 60)
    torch_tensors_close("output", nn.AdaptiveAvgPool2d(1)(inputs), DaceModule(nn.AdaptiveAvgPool2d(1))(inputs.cuda()).cpu())
    # ... :12-33 in inference form (the reference's test runs BatchNorm2d in training mode, which is not provided here)
    bn = nn.BatchNorm2d(64).eval()
    with torch.no_grad():
        bn.running_mean.normal_()
        bn.running_var.uniform_(0.5, 2.0)
    torch_tensors_close("output", bn(inputs), DaceModule(bn)(inputs.cuda()).cpu())
    with pytest.raises(NotImplementedError, match="inference only"):
        DaceModule(nn.BatchNorm2d(64), training=True)


class _PadConv(nn.Module):
    """tests/transformation/test_pad_conv_fusion.py:13-20 of the reference."""
    def __init__(self):
        super().__init__()
        self.conv = nn.Conv2d(3, 6, kernel_size=(3, 3))

    def forward(self, x):
        return self.conv(torch.nn.functional.pad(x, [2, 2]))


class _ConvPoolViewRelu(nn.Module):
    """tests/transformation/test_reshape_elimination.py:12-20 of the reference."""
    def __init__(self):
        super().__init__()
        self.conv = nn.Conv2d(6, 16, 5)

    def forward(self, x):
        F = torch.nn.functional
        x = F.max_pool2d(F.relu(self.conv(x)), 2)
        return F.relu(x.view(-1, 256))


class _AddTwo(nn.Module):
    """tests/transformation/test_input_to_constant.py:13-19 of the reference (an unused parameter, a scalar constant)."""
    def __init__(self):
        super().__init__()
        self.fc1 = nn.Linear(5, 3)

    def forward(self, x):
        return x + 2


_TRANSFORMATION_TEST_MODULES = [(_PadConv, (4, 3, 24, 24), ["mi355x_conv2d_f32"]),
                                (_ConvPoolViewRelu, (100, 6, 12, 12), ["mi355x_conv2d_f32", "mi355x_maxpool2d_f32", "mi355x_eltwise_f32"]),
                                (_AddTwo, (10, 5), ["mi355x_eltwise_f32"])]


@pytest.mark.parametrize("cls, shape, launches", _TRANSFORMATION_TEST_MODULES)
def test_transformation_test_modules_launch_lists(cls, shape, launches):
    # the exporter's pad arithmetic (a dozen shape nodes) folds to a constant, the Pad into the convolution's pads --
    # the output's symbolic declared shape is replaced by the inferred one; views cost nothing
    dm = DaceModule(cls(), dummy_inputs=(torch.rand(*shape), ))
    assert _functions(dm) == launches
    if cls is _PadConv:
        call = [n for n, _ in dm.dace_model.sdfg.all_nodes_recursive() if isinstance(n, dace.KernelCall)][0]
        assert [0, 2, 0, 2] in [getattr(a, "values", None) for a in call.args]


@pytest.mark.gpu
@pytest.mark.parametrize("cls, shape, launches", _TRANSFORMATION_TEST_MODULES)
def test_transformation_test_modules_results(cls, shape, launches):
    torch.manual_seed(8)
    torch_module = cls()
    dace_module = DaceModule(copy.deepcopy(torch_module))
    input = torch.rand(*shape)
    torch_tensors_close("output", torch_module(input), dace_module(input.cuda()).cpu())


class _TwoConvs(nn.Module):
    """tests/pytorch/test_conv2d.py:12-21 of the reference."""
    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(1, 4, 3)
        self.conv2 = nn.Conv2d(4, 4, 3)

    def forward(self, x):
        x = torch.relu(self.conv1(x))
        return torch.relu(self.conv2(x))


@pytest.mark.gpu
def test_conv2d_wrapped_and_decorated(sdfg_name):
    # tests/pytorch/test_conv2d.py:11-38
    torch.manual_seed(9)
    ptmodel = _TwoConvs()
    x = torch.rand(1, 1, 8, 8)

    @dace_module(sdfg_name=sdfg_name)
    class TestDecorator(_TwoConvs):
        pass

    dace_model = DaceModule(ptmodel, sdfg_name=sdfg_name + "_wrapped")
    dace_output = dace_model(x.cuda())
    decorated = TestDecorator()
    decorated_output = decorated(x.cuda())
    assert np.allclose(ptmodel(x).detach().numpy(), dace_output.cpu().numpy(), atol=1e-06)
    assert np.allclose(decorated.model(x).detach().numpy(), decorated_output.cpu().numpy(), atol=1e-06)


@pytest.mark.gpu
def test_debug_transients_decorator():
    # tests/pytorch/test_debug_transients.py:8-23: the intermediate comes back as a second output
    @dace_module(debug_transients=True)
    class Module(nn.Module):
        def forward(self, x):
            y = x + 3
            return y * 5

    module = Module()
    x = torch.rand(5, 5)
    output, y = module(x.cuda())
    torch_tensors_close("output", (x + 3) * 5, output.cpu())
    torch_tensors_close("y", x + 3, y.cpu())


class _LogSqrt(nn.Module):
    """The example of the reference's DaceModule docstring (daceml/pytorch/module.py:43-55)."""
    def forward(self, x):
        x = torch.log(x)
        x = torch.sqrt(x)
        return x


def test_docstring_example_is_one_launch():
    dm = DaceModule(_LogSqrt(), dummy_inputs=(torch.ones(2), ))
    assert [n.op_type for n in dm.onnx_model.graph.node] == ["Log", "Sqrt"]
    assert _functions(dm) == ["mi355x_eltwise_program_f32"]


@pytest.mark.gpu
def test_docstring_example_result():
    dace_module = DaceModule(_LogSqrt())
    assert dace_module(torch.ones(2).cuda()).tolist() == [0.0, 0.0]
    x = torch.rand(7, 5) + 1.0
    assert torch.allclose(dace_module.model(x), DaceModule(_LogSqrt())(x.cuda()).cpu(), rtol=1e-6, atol=1e-7)


class _ResidualBlock(nn.Module):
    """A ResNet basic block with a projection shortcut (not a Sequential: only the exporter can write it)."""
    def __init__(self, c):
        super().__init__()
        self.c1, self.b1 = nn.Conv2d(c, c, 3, padding=1, bias=False), nn.BatchNorm2d(c)
        self.c2, self.b2 = nn.Conv2d(c, c, 3, padding=1, bias=False), nn.BatchNorm2d(c)
        self.down = nn.Sequential(nn.Conv2d(c, c, 1, bias=False), nn.BatchNorm2d(c))

    def forward(self, x):
        h = torch.relu(self.b1(self.c1(x)))
        return torch.relu(self.b2(self.c2(h)) + self.down(x))


def _residual_block():
    torch.manual_seed(6)
    net = _ResidualBlock(16).eval()
    with torch.no_grad():
        for m in net.modules():
            if isinstance(m, nn.BatchNorm2d):
                m.running_mean.normal_(std=0.3)
                m.running_var.uniform_(0.5, 2.0)
                m.weight.normal_(1.0, 0.2)
                m.bias.normal_(std=0.2)
    return net


def test_residual_block_launch_list():
    dm = DaceModule(_residual_block(), dummy_inputs=(torch.randn(2, 16, 8, 8), ))
    assert [n.op_type for n in dm.onnx_model.graph.node] == ["Conv", "BatchNormalization", "Relu", "Conv", "BatchNormalization",
                                                             "Conv", "BatchNormalization", "Add", "Relu"]
    # three convolutions with their normalizations inside; the first takes its ReLU, the last to run takes the
    # other branch as its residual and the ReLU after the sum (bias | residual | relu-after = 25)
    calls = [n for n, _ in dm.dace_model.expand().all_nodes_recursive() if isinstance(n, dace.KernelCall)]
    assert sorted(c.function for c in calls) == ["mi355x_conv2d_f32"] * 2 + ["mi355x_conv2d_res_f32"]
    assert [c.args[-2] for c in calls if c.function == "mi355x_conv2d_res_f32"] == [25]
    assert sorted(c.args[-2] for c in calls if c.function == "mi355x_conv2d_f32") == [1, 3]


@pytest.mark.gpu
def test_residual_block_results():
    net = _residual_block()
    x = torch.randn(3, 16, 8, 8)
    with torch.no_grad():
        ref = copy.deepcopy(net).double()(x.double())
    assert rel_err(ref.numpy(), DaceModule(net)(x.cuda()).cpu().numpy()) < FP32_REL_TOL
    assert rel_err(ref.numpy(), DaceModule(net, auto_optimize=False)(x.cuda()).cpu().numpy()) < FP32_REL_TOL


# ----------------------------------------------------------------------------- the TorchScript exporter path
class _TwoInputNet(nn.Module):
    """Not a Sequential and with two inputs: only the exporter can turn it into a graph."""
    def __init__(self):
        super().__init__()
        self.conv = nn.Conv2d(3, 8, 3, padding=1)
        self.fc = nn.Linear(8 * 8 * 8, 12)

    def forward(self, x, y):
        h = torch.relu(self.conv(x)) + y
        return torch.softmax(self.fc(h.flatten(1)), dim=-1)


def test_exporter_path_writes_the_reference_flavoured_graph():
    from dace_onnx_amd.onnx import proto
    from dace_onnx_amd.pytorch.module import export_with_torch
    layer = _bert_layer(128, 2, 256)
    m = proto.parse_model(export_with_torch(layer, (torch.randn(2, 128, 128), )))
    ops = {n.op_type for n in m.graph.node}
    # no constant folding by the exporter: shape arithmetic and weight transposes are nodes
    assert {"Unsqueeze", "Concat", "Constant", "Transpose", "MatMul", "Erf", "ReduceMean"} <= ops
    names = {t.name for t in m.graph.initializer}
    assert {"attention.self.query.weight", "output.dense.weight", "output.LayerNorm.bias"} <= names
    assert names <= {i.name for i in m.graph.input}          # keep_initializers_as_inputs
    # imported with constant folding, fused: the same seven launches as the structural graph, and the three
    # [N, K] projection weights concatenated along N without a transposed copy
    dm = DaceModule(layer, dummy_inputs=(torch.randn(2, 128, 128), ), exporter="torch")
    assert sorted(_functions(dm)) == ["mi355x_attention_f32"] + ["mi355x_gemm_f32"] * 4 + ["mi355x_layernorm_f32"] * 2
    assert tuple(dm.dace_model.weights["attention.self.query.weight_hcat"].shape) == (3 * 128, 128)
    assert not any(k.endswith("_kcontig") for k in dm.dace_model.weights)
    with pytest.raises(ValueError, match="exporter must be"):
        DaceModule(layer, exporter="onnxruntime")


def test_auto_falls_back_to_the_exporter():
    net = _TwoInputNet().eval()
    with pytest.raises(UnsupportedModule):
        DaceModule(net, dummy_inputs=(torch.randn(2, 3, 8, 8), torch.randn(2, 8, 8, 8)), exporter="structural")
    dm = DaceModule(net, dummy_inputs=(torch.randn(2, 3, 8, 8), torch.randn(2, 8, 8, 8)))
    assert len(dm.dace_model.inputs) == 2
    # relu(conv(x)) + y: ReLU and the second input both ride in the convolution's epilogue
    assert _functions(dm) == ["mi355x_conv2d_res_f32", "mi355x_gemm_f32", "mi355x_softmax_f32"]


@pytest.mark.gpu
def test_exporter_path_results():
    torch.manual_seed(3)
    net = _TwoInputNet().eval()
    x, y = torch.randn(4, 3, 8, 8), torch.randn(4, 8, 8, 8)
    with torch.no_grad():
        ref = copy.deepcopy(net).double()(x.double(), y.double())
    got = DaceModule(net)(x.cuda(), y.cuda())
    assert rel_err(ref.numpy(), got.cpu().numpy()) < FP32_REL_TOL

    layer = _bert_layer(128, 2, 256)
    with torch.no_grad():
        for p in layer.parameters():      # the default initialisation leaves biases at zero
            p.add_(torch.randn_like(p) * 0.02)
    h = torch.randn(3, 128, 128)
    with torch.no_grad():
        ref = copy.deepcopy(layer).double()(h.double())
        ref = ref[0] if isinstance(ref, (tuple, list)) else ref
    for exporter in ("torch", "structural"):
        got = DaceModule(layer, exporter=exporter)(h.cuda())
        assert rel_err(ref.numpy(), got.cpu().numpy()) < FP32_REL_TOL, exporter


def test_multihead_attention_launch_list():
    # the module of the reference's tests/pytorch/test_attn.py, small: the exporter's 76 nodes (Shape, Gather,
    # Slice of the packed in_proj_weight, Unsqueeze, Concat ...) fold to MatMul / Transpose / Reshape / Mul /
    # Softmax / ReduceMean; the query scale moves into the GEMM's alpha, the transposes into operand strides
    mha = nn.MultiheadAttention(256, 4, bias=False).eval()
    q, k, v = torch.randn(128, 2, 256), torch.randn(128, 2, 256), torch.randn(128, 2, 256)
    dm = DaceModule(mha, dummy_inputs=(q, k, v))
    assert dm.dace_model.inputs == ["query", "key", "value"] and len(dm.dace_model.outputs) == 2
    assert _functions(dm) == ["mi355x_gemm_f32"] * 4 + ["mi355x_softmax_f32"] + ["mi355x_gemm_f32"] * 2 + \
        ["mi355x_reduce_mean_f32"]


@pytest.mark.gpu
def test_multihead_attention_module():
    # tests/pytorch/test_attn.py at its own sizes: B=2, 16 heads of 64, 512 queries and keys, both outputs
    torch.manual_seed(4)
    B, H, P, S = 2, 16, 64, 512
    N = P * H
    k, q, v = torch.randn(S, B, N), torch.randn(S, B, N), torch.randn(S, B, N)
    mha = nn.MultiheadAttention(N, H, bias=False).eval()
    with torch.no_grad():
        ref_out, ref_weights = copy.deepcopy(mha).double()(q.double(), k.double(), v.double())
    out, weights = DaceModule(mha)(q.cuda(), k.cuda(), v.cuda())
    torch_tensors_close("outputs_0", ref_out.float(), out.cpu(), rtol=1e-4, atol=1e-5)
    torch_tensors_close("outputs_1", ref_weights.float(), weights.cpu(), rtol=1e-4, atol=1e-6)
    assert rel_err(ref_out.numpy(), out.cpu().numpy()) < FP32_REL_TOL
    assert rel_err(ref_weights.numpy(), weights.cpu().numpy()) < FP32_REL_TOL


def test_hooks_run_in_order_and_can_change_the_graph():
    # daceml/pytorch/module.py:83-210: named hooks after the ONNX import and after compilation
    m = nn.Sequential(nn.Linear(8, 16), nn.ReLU(), nn.Linear(16, 4)).eval()
    seen = []
    dm = DaceModule(m)
    assert list(dm.post_onnx_hooks) == ["auto_optimize"]
    dm.append_post_onnx_hook("after", lambda mod: seen.append(("after", len(_functions(mod)))))
    dm.prepend_post_onnx_hook("before", lambda mod: seen.append(
        ("before", sorted(type(n).__name__ for n in mod.sdfg.states()[0].nodes() if type(n).__name__.startswith("ONNX")))))
    dm.append_post_onnx_hook("after", lambda mod: seen.append(("after_1", None)))      # same name: made unique
    assert list(dm.post_onnx_hooks) == ["before", "auto_optimize", "after", "after_1"]
    dm.function = dm._initialize_sdfg((torch.randn(5, 8), ))
    # "before" saw the imported ONNX nodes, "after" the fused and expanded graph: two GEMM launches
    assert seen == [("before", ["ONNXGemm", "ONNXGemm", "ONNXRelu"]), ("after", 2), ("after_1", None)]
    # without the optimisation hook the graph is expanded node by node on the first call
    plain = DaceModule(m, dummy_inputs=(torch.randn(5, 8), ), auto_optimize=False)
    assert list(plain.post_onnx_hooks) == [] and not plain.dace_model._expanded


@pytest.mark.gpu
def test_debug_transients_and_compile_hook():
    torch.manual_seed(5)
    m = nn.Sequential(nn.Linear(8, 16), nn.ReLU(), nn.Linear(16, 4)).eval()
    x = torch.randn(5, 8)
    compiled = []
    dm = DaceModule(m, debug_transients=True)
    dm.append_post_compile_hook("record", compiled.append)
    outs = dm(x.cuda())
    # the module's output first, then every intermediate (here: the two values between the three nodes)
    assert isinstance(outs, tuple) and len(outs) == 3 and len(compiled) == 1 and compiled[0].num_launches == 3
    with torch.no_grad():
        h = m[0](x)
        expected = [m(x), h, torch.relu(h)]
    for got, ref in zip(outs, expected):
        assert rel_err(ref.numpy(), got.cpu().numpy()) < FP32_REL_TOL
    dm(x.cuda())
    assert len(compiled) == 1          # compiled once

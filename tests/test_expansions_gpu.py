"""GPU parity of every "mi355x" expansion against the oracle, through the same
graph-building code the reference's expansion tests use
(tests/pure_expansions/test_expansions.py, test_conv_expansion.py,
tests/test_python_frontend.py): build a one-node SDFG (or use the frontend call
form), expand, check that the node really became a kernel call, run, compare.

Tolerance: fp32 kernels within 1e-4 of the expected tensor's largest magnitude
(FP32_REL_TOL); MatMulInteger bit-exact.
"""
import numpy as np
import pytest
import torch

from dace_onnx_amd import _lib, sdfg as dace
import dace_onnx_amd.onnx as donnx
from dace_onnx_amd.onnx import proto
from dace_onnx_amd.util import utils
from oracle import pure_ops as O
from conftest import rel_err, FP32_REL_TOL

pytestmark = pytest.mark.gpu


def assert_expanded_to_kernels(sdfg):
    # the reference asserts a MapEntry exists, i.e. the node did not go to ONNX Runtime
    assert any(isinstance(n, (dace.KernelCall, dace.AliasNode)) for n, _ in sdfg.all_nodes_recursive())
    assert not any(isinstance(n, dace.LibraryNode) for n, _ in sdfg.all_nodes_recursive())


# ----------------------------------------------------------------------------- MatMul / Gemm
@pytest.mark.parametrize("a_shape, b_shape", [([2, 4], [4, 3]), ([8, 12, 128, 64], [8, 12, 64, 128]),
                                              ([8, 128, 768], [768, 3072]), ([3, 5, 7], [7, 2]), ([5, 7], [3, 7, 2]),
                                              ([2, 1, 33, 65], [3, 65, 17]), ([1, 1], [1, 1]), ([130, 131], [131, 129])])
def test_matmul_expansion(a_shape, b_shape, sdfg_name):
    sdfg = dace.SDFG(sdfg_name)
    rng = np.random.default_rng(0)
    X = rng.random(a_shape).astype(np.float32)
    Z = rng.random(b_shape).astype(np.float32)
    expected_result = O.matmul(X, Z)
    sdfg.add_array("X", a_shape, dace.float32)
    sdfg.add_array("Z", b_shape, dace.float32)
    sdfg.add_array("__return", expected_result.shape, dace.float32)
    state = sdfg.add_state()
    access_X = state.add_access("X")
    access_Z = state.add_access("Z")
    access_result = state.add_access("__return")
    op_node = donnx.ONNXMatMul("Matmul")
    state.add_node(op_node)
    state.add_edge(access_X, None, op_node, "A", sdfg.make_array_memlet("X"))
    state.add_edge(access_Z, None, op_node, "B", sdfg.make_array_memlet("Z"))
    state.add_edge(op_node, "Y", access_result, None, sdfg.make_array_memlet("__return"))
    sdfg.expand_library_nodes()
    assert_expanded_to_kernels(sdfg)
    result = sdfg(X=X, Z=Z)
    assert np.allclose(expected_result, result)  # the reference's check (test_expansions.py:56)
    assert rel_err(X.astype(np.float64) @ Z.astype(np.float64), result) < FP32_REL_TOL


def test_matmul_python_frontend_form():
    # tests/test_python_frontend.py:12-22
    rng = np.random.default_rng(1)
    A = rng.normal(size=(5, 5)).astype(np.float32)
    B = rng.normal(size=(5, 3)).astype(np.float32)
    out = np.zeros((5, 3), np.float32)
    donnx.ONNXMatMul(A=A.copy(), B=B.copy(), Y=out)
    assert np.allclose(A @ B, out)
    with pytest.raises(TypeError, match="Unknown arguments"):
        donnx.ONNXMatMul(A=A, B=B, Y=out, Q=out)


@pytest.mark.parametrize("transA, transB, alpha, c_shape", [(0, 1, 1.0, (9, )), (0, 0, 1.0, None), (1, 0, 0.5, (1, 9)),
                                                            (1, 1, 2.0, (10, 9)), (0, 1, 1.0, None)])
def test_gemm(transA, transB, alpha, c_shape):
    rng = np.random.default_rng(2)
    M, K, N = 10, 12, 9
    A = rng.normal(size=(K, M) if transA else (M, K)).astype(np.float32)
    B = rng.normal(size=(N, K) if transB else (K, N)).astype(np.float32)
    C = rng.normal(size=c_shape).astype(np.float32) if c_shape else None
    Y = np.zeros((M, N), np.float32)
    kwargs = dict(A=A, B=B, Y=Y, transA=transA, transB=transB, alpha=alpha)
    if C is not None:
        kwargs["C"] = C
    donnx.ONNXGemm(**kwargs)
    assert rel_err(O.gemm(A, B, C, alpha=alpha, transA=transA, transB=transB), Y) < FP32_REL_TOL


# ----------------------------------------------------------------------------- Conv
@pytest.mark.parametrize("num_in_channels, kernel_size, num_filters, bias",
                         [(1, (3, 3), 8, True), (8, (3, 3), 3, False), (8, (5, 5), 3, True), (8, (4, 4), 3, False)])
def test_conv_simple(num_in_channels, kernel_size, num_filters, bias):
    # the reference's grid (test_conv_expansion.py:10-64), frontend call form
    batch_size = 8
    rng = np.random.default_rng(3)
    X = rng.random((batch_size, num_in_channels, 32, 32)).astype(np.float32)
    W = rng.random((num_filters, num_in_channels, *kernel_size)).astype(np.float32)
    B = rng.random(num_filters).astype(np.float32) if bias else None
    expected = O.conv2d(X, W, B)
    dace_Z = np.zeros_like(expected)
    if bias:
        donnx.ONNXConv(X=X, W=W, B=B, Y=dace_Z)
    else:
        donnx.ONNXConv(X=X, W=W, Y=dace_Z)
    assert np.allclose(expected, dace_Z, rtol=1e-4, atol=1e-4)
    assert rel_err(expected, dace_Z) < FP32_REL_TOL


def test_conv_config1_stride2():
    # benchmark config 1 (5x3x10x10 input, 16 filters 3x3, stride 2) and the reference's README example (examples/plot_conv.py:43-46)
    rng = np.random.default_rng(1)
    X = rng.random((5, 3, 10, 10), dtype=np.float32)
    W = rng.random((16, 3, 3, 3), dtype=np.float32)
    Y = np.zeros((5, 16, 4, 4), np.float32)
    donnx.ONNXConv(X=X, W=W, Y=Y, strides=[2, 2])
    assert rel_err(O.conv2d(X, W, strides=(2, 2)), Y) < FP32_REL_TOL


@pytest.mark.parametrize("shape, wshape, attrs", [
    ((2, 5, 13, 17), (7, 5, 3, 2), dict(pads=[1, 2, 0, 1], strides=[2, 1], dilations=[2, 3])),
    ((1, 3, 7, 7), (20, 3, 7, 7), dict()),                                     # output 1x1
    ((3, 4, 9, 9), (65, 4, 1, 1), dict(strides=[3, 3])),                       # 1x1 kernel, odd filter count
    ((2, 6, 15, 14), (33, 6, 3, 3), dict(auto_pad="SAME_UPPER", strides=[2, 2])),
    ((1, 2, 30, 31), (4, 2, 5, 3), dict(pads=[2, 1, 2, 1])),                   # OH*OW % 4 != 0: scalar stores
    # C*KH*KW % 32 == 0: the transposed-gather kernel (64 x 64 and 64 x 128 position tiles, ragged edges)
    ((2, 32, 12, 12), (64, 32, 3, 3), dict(pads=[1, 1, 1, 1])),
    ((3, 32, 9, 11), (70, 32, 1, 1), dict()),                                  # K = 32: a single k tile, 70 filters
    ((2, 8, 14, 13), (5, 8, 2, 2), dict(pads=[0, 1, 1, 0], strides=[2, 1], dilations=[1, 2])),   # odd OH*OW
    ((40, 16, 30, 30), (48, 16, 3, 2), dict(pads=[2, 0, 1, 3], strides=[1, 2])),                 # many tiles -> 128-wide
    ((1, 64, 5, 5), (64, 64, 3, 3), dict(auto_pad="SAME_UPPER")),              # K = 576, 25 positions
])
def test_conv_attributes(shape, wshape, attrs):
    rng = np.random.default_rng(4)
    X = rng.normal(size=shape).astype(np.float32)
    W = rng.normal(size=wshape).astype(np.float32)
    B = rng.normal(size=wshape[0]).astype(np.float32)
    strides = tuple(attrs.get("strides", (1, 1)))
    dil = tuple(attrs.get("dilations", (1, 1)))
    if attrs.get("auto_pad") == "SAME_UPPER":
        pads = []
        for size, s, k in ((shape[2], strides[0], wshape[2]), (shape[3], strides[1], wshape[3])):
            total = max((-(-size // s) - 1) * s + k - size, 0)
            pads.append((total // 2, total - total // 2))
        pads = (pads[0][0], pads[1][0], pads[0][1], pads[1][1])
    else:
        pads = tuple(attrs.get("pads", (0, 0, 0, 0)))
    expected = O.conv2d(X, W, B, strides, pads, dil)
    Y = np.zeros_like(expected)
    donnx.ONNXConv(X=X, W=W, B=B, Y=Y, **attrs)
    assert rel_err(expected, Y) < FP32_REL_TOL


# ----------------------------------------------------------------------------- Softmax / LayerNorm
@pytest.mark.parametrize("axis", [0, -1])
def test_softmax(axis, sdfg_name):
    # tests/pure_expansions/test_expansions.py:345-379
    X = np.random.default_rng(5).normal(scale=10, size=(2, 4, 10)).astype(np.float32)
    torch_result = torch.nn.functional.softmax(torch.Tensor(X), dim=axis).numpy()
    sdfg = dace.SDFG(sdfg_name)
    sdfg.add_array("X", [2, 4, 10], dace.float32)
    sdfg.add_array("__return", torch_result.shape, dace.float32)
    state = sdfg.add_state()
    access_X = state.add_access("X")
    access_result = state.add_access("__return")
    op_node = donnx.ONNXSoftmax("softmax")
    op_node.axis = axis
    state.add_node(op_node)
    state.add_edge(access_X, None, op_node, "input", sdfg.make_array_memlet("X"))
    state.add_edge(op_node, "output", access_result, None, sdfg.make_array_memlet("__return"))
    sdfg.expand_library_nodes()
    assert_expanded_to_kernels(sdfg)
    result = sdfg(X=X)
    assert np.linalg.norm(torch_result - result) < 1e-5
    assert rel_err(O.softmax(X, axis=axis), result) < FP32_REL_TOL


@pytest.mark.parametrize("shape", [(8, 12, 16, 128), (7, 64), (33, 256), (5, 1000), (3, 2048), (2, 5000), (4, 36),
                                   (3, 1), (5, 7), (2, 130)])
def test_softmax_row_lengths(shape):
    X = np.random.default_rng(6).normal(scale=4, size=shape).astype(np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXSoftmax(input=X, output=Y, axis=-1)
    assert rel_err(O.softmax(X), Y) < FP32_REL_TOL
    assert np.allclose(Y.sum(-1), 1.0, atol=1e-5)


def test_softmax_large_values_and_middle_axis():
    X = np.array([[1000.0, 999.0, -1000.0, 0.0]] * 3, np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXSoftmax(input=X, output=Y, axis=1)
    assert np.isfinite(Y).all() and rel_err(O.softmax(X), Y) < FP32_REL_TOL
    X = np.random.default_rng(7).normal(size=(3, 17, 5, 9)).astype(np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXSoftmax(input=X, output=Y, axis=1)
    assert rel_err(O.softmax(X, axis=1), Y) < FP32_REL_TOL


@pytest.mark.parametrize("shape, axis", [((8, 16, 768), -1), ((5, 256), -1), ((3, 1000), 1), ((2, 4096), -1),
                                         ((2, 5000), -1), ((3, 30), -1), ((4, 6, 48), 1), ((3, 1), -1)])
def test_layer_normalization(shape, axis):
    rng = np.random.default_rng(8)
    X = rng.normal(size=shape).astype(np.float32)
    norm_shape = shape[axis % len(shape):]
    g = rng.normal(1.0, 0.02, size=norm_shape).astype(np.float32)
    b = rng.normal(0.0, 0.02, size=norm_shape).astype(np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXLayerNormalization(X=X, Scale=g, B=b, Y=Y, axis=axis, epsilon=1e-12)
    assert rel_err(O.layer_normalization(X, g, b, axis=axis, epsilon=1e-12), Y) < FP32_REL_TOL
    Y2 = np.zeros_like(X)
    donnx.ONNXLayerNormalization(X=X, Scale=g, Y=Y2, axis=axis)  # no bias, default epsilon
    assert rel_err(O.layer_normalization(X, g, None, axis=axis, epsilon=1e-5), Y2) < FP32_REL_TOL


@pytest.mark.parametrize("waves", [None, 2, 3])
@pytest.mark.parametrize("batch, sq", [((2, 3), 128), ((1, 5), 100), ((4, ), 16), ((1, 1), 1)])
def test_fused_attention_c_abi(tuning, batch, sq, waves):
    # softmax(scale * Q K^T) V through the C ABI, operands as strided slices of one packed projection; with the
    # library's 64 query rows per workgroup and with the 32- and 48-row forms MI355X_ATTN_WAVES selects
    tuning(MI355X_ATTN_WAVES=waves)
    rng = np.random.default_rng(31)
    b0, b1 = (1, ) * (2 - len(batch)) + tuple(batch)
    packed = torch.from_numpy(rng.normal(size=(b0, max(sq, 128), b1, 3, 64)).astype(np.float32)).cuda()
    q, k, v = packed[:, :sq, :, 0], packed[:, :128, :, 1], packed[:, :128, :, 2]      # [b0, S, b1, 64] views
    out = torch.zeros(b0, sq, b1, 64, device="cuda")
    lib = _lib.library()
    strides = lambda t: _lib.i64_array([t.stride(0), t.stride(2), t.stride(1)])
    scale = 0.125
    _lib.check(lib.mi355x_attention_f32(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), b0, b1, sq, 128, 64,
                                        strides(q), strides(k), strides(v), strides(out), scale, _lib.current_stream()),
               "mi355x_attention_f32")
    Q, K, V = (t.permute(0, 2, 1, 3).cpu().numpy().astype(np.float64) for t in (q, k, v))
    expected = O.matmul(O.softmax(O.matmul(Q, np.swapaxes(K, -1, -2)) * scale, axis=-1), V)
    assert rel_err(expected, out.permute(0, 2, 1, 3).cpu().numpy()) < FP32_REL_TOL
    # another head size is rejected, nothing is launched
    assert lib.mi355x_attention_f32(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), b0, b1, sq, 128, 32,
                                    strides(q), strides(k), strides(v), strides(out), scale, _lib.current_stream()) == 1


@pytest.mark.parametrize("sk", [1, 5, 64, 127, 129, 200, 256, 384, 1000])
def test_fused_attention_any_number_of_keys(sk):
    # keys walked in blocks of 128 with a running row maximum and sum; the last block may be ragged.
    # Scores with a large spread (scale 1) so that the running maximum really moves between blocks.
    rng = np.random.default_rng(sk)
    b0, b1, sq = 2, 3, 70
    q = torch.from_numpy(rng.normal(size=(b0, b1, sq, 64)).astype(np.float32)).cuda()
    k = torch.from_numpy(rng.normal(size=(b0, b1, sk, 64)).astype(np.float32)).cuda()
    v = torch.from_numpy(rng.normal(size=(b0, b1, sk, 64)).astype(np.float32)).cuda()
    out = torch.full((b0, b1, sq, 64), float("nan"), device="cuda")
    strides = lambda t: _lib.i64_array([t.stride(0), t.stride(1), t.stride(2)])
    _lib.check(_lib.library().mi355x_attention_f32(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), b0, b1, sq,
                                                   sk, 64, strides(q), strides(k), strides(v), strides(out), 1.0,
                                                   _lib.current_stream()), "mi355x_attention_f32")
    Q, K, V = (t.cpu().numpy().astype(np.float64) for t in (q, k, v))
    expected = O.matmul(O.softmax(O.matmul(Q, np.swapaxes(K, -1, -2)), axis=-1), V)
    got = out.cpu().numpy()
    assert not np.isnan(got).any() and rel_err(expected, got) < FP32_REL_TOL


# ----------------------------------------------------------------------------- elementwise
@pytest.mark.parametrize("a_shape, b_shape", [((8, 16, 768), (768, )), ((8, 16, 768), (8, 16, 768)), ((5, 1, 7), (3, 1)),
                                              ((4, 6), ()), ((1, ), (2, 3, 4)), ((768, ), (2, 4, 768)), ((3, 5), (3, 1))])
@pytest.mark.parametrize("op", ["Add", "Sub", "Mul", "Div"])
def test_binary_broadcast(op, a_shape, b_shape):
    rng = np.random.default_rng(9)
    A = rng.normal(size=a_shape).astype(np.float32)
    B = (rng.random(size=b_shape) + 0.5).astype(np.float32)
    expected = getattr(O, op.lower())(A, B)
    C = np.zeros(expected.shape, np.float32)
    getattr(donnx, "ONNX" + op)(A=A, B=B, C=C)
    assert np.array_equal(expected, C) or rel_err(expected, C) < 1e-6


def test_gelu_dense_grid_absolute_error():
    """The kernel's own erf (a fit, not the library routine) against the double-precision closed form on a
    dense grid: the absolute error of Gelu stays within two fp32 roundings of the result."""
    import math
    X = np.linspace(-8.0, 8.0, 400001).astype(np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXGelu(X=X, Y=Y)
    x64 = X.astype(np.float64)
    ref = 0.5 * x64 * (1.0 + np.vectorize(math.erf)(x64 / math.sqrt(2.0)))
    err = np.abs(Y.astype(np.float64) - ref)
    assert err.max() <= 2 * np.spacing(np.float32(8.0)), err.max()
    assert (err[np.abs(X) <= 1.0]).max() <= 2.5e-7
    assert np.abs(Y[X <= -6.0]).max() <= 1e-6      # left tail goes to zero, not to garbage
    assert Y[X == 0.0][0] == 0.0


@pytest.mark.parametrize("shape", [(8, 16, 3072), (7, ), (1, 3, 5), (4097, )])
def test_unary_ops(shape):
    X = np.random.default_rng(10).normal(scale=2, size=shape).astype(np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXRelu(X=X, Y=Y)
    assert np.array_equal(O.relu(X), Y)
    donnx.ONNXGelu(X=X, Y=Y)
    assert rel_err(O.gelu(X), Y) < FP32_REL_TOL
    donnx.ONNXErf(input=X, output=Y)
    assert rel_err(O.erf(X), Y) < FP32_REL_TOL
    donnx.ONNXSqrt(X=np.abs(X), Y=Y)
    assert rel_err(O.sqrt(np.abs(X)), Y) < 1e-6


@pytest.mark.parametrize("shape", [(8, 16, 3072), (7, ), (1, 3, 5), (4097, )])
@pytest.mark.parametrize("op, conns, positive", [("Log", ("input", "output"), True), ("Tanh", ("input", "output"), False),
                                                 ("Exp", ("input", "output"), False), ("Sigmoid", ("X", "Y"), False),
                                                 ("Softplus", ("X", "Y"), False), ("Reciprocal", ("X", "Y"), True),
                                                 ("Neg", ("X", "Y"), False), ("Abs", ("X", "Y"), False)])
def test_more_unary_ops(op, conns, positive, shape):
    """The unary maps of pure_implementations.py:23-38, 275-298, 696-712 (and Exp, Neg, Abs): every element
    within a few fp32 roundings of the oracle's value."""
    X = np.random.default_rng(31).normal(scale=3, size=shape).astype(np.float32)
    if positive:
        X = np.abs(X) + np.float32(0.05)
    Y = np.zeros_like(X)
    getattr(donnx, "ONNX" + op)(**{conns[0]: X, conns[1]: Y})
    expected = getattr(O, op.lower())(X)
    if op in ("Neg", "Abs"):
        assert np.array_equal(expected, Y)
    else:
        assert np.allclose(Y, expected, rtol=2e-6, atol=2e-7), np.abs(Y - expected).max()


def test_softplus_sigmoid_extremes():
    """Same behaviour as the reference's formulas at the ends: log(1 + exp(x)) overflows where exp does and
    is exactly 0 far to the left; the sigmoid saturates at 0 and 1 without NaN."""
    X = np.array([-200.0, -104.0, -20.0, 0.0, 20.0, 88.0, 89.0, 200.0], dtype=np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXSoftplus(X=X, Y=Y)
    expected = O.softplus(X)
    assert np.array_equal(np.isinf(expected), np.isinf(Y)) and np.allclose(Y[:-2], expected[:-2], rtol=2e-6, atol=1e-7)
    donnx.ONNXSigmoid(X=X, Y=Y)
    assert not np.isnan(Y).any() and Y[0] == 0.0 and Y[-1] == 1.0 and Y[3] == 0.5
    assert np.allclose(Y, O.sigmoid(X), rtol=2e-6, atol=1e-30)


@pytest.mark.parametrize("shape, axes, keepdims", [((8, 16, 768), [-1], 1), ((5, 33), [1], 0), ((4, 6, 10), [1], 1),
                                                   ((3, 4, 5, 6), [1, 2], 0), ((7, 9), [0, 1], 1), ((2, 4100), [-1], 1)])
def test_reduce_mean(shape, axes, keepdims):
    X = np.random.default_rng(15).normal(1.0, 2.0, size=shape).astype(np.float32)
    expected = O.reduce_mean(X.astype(np.float64), axes, keepdims)
    Y = np.zeros(expected.shape, np.float32)
    donnx.ONNXReduceMean(data=X, reduced=Y, axes=axes, keepdims=keepdims)
    assert rel_err(expected, Y) < FP32_REL_TOL


@pytest.mark.parametrize("shape, axes, keepdims", [((8, 16, 768), [-1], 1), ((5, 33), [1], 0), ((4, 6, 10), [1], 1),
                                                   ((3, 4, 5, 6), [1, 2], 0), ((7, 9), [0, 1], 1), ((2, 4100), [-1], 1),
                                                   ((4100, 3), [0], 0)])
@pytest.mark.parametrize("op", ["ReduceSum", "ReduceMax", "ReduceMin"])
def test_reduce_sum_max_min(op, shape, axes, keepdims):
    """np.sum / np.max / np.min over ``axes`` (pure_implementations.py:301-343): extrema exact, sums against
    the double-precision sum."""
    X = np.random.default_rng(17).normal(1.0, 2.0, size=shape).astype(np.float32)
    oracle = {"ReduceSum": O.reduce_sum, "ReduceMax": O.reduce_max, "ReduceMin": O.reduce_min}[op]
    expected = oracle(X.astype(np.float64), axes, keepdims)
    Y = np.zeros(expected.shape, np.float32)
    getattr(donnx, "ONNX" + op)(data=X, reduced=Y, axes=axes, keepdims=keepdims)
    if op == "ReduceSum":
        assert rel_err(expected, Y) < FP32_REL_TOL
        abs_sum = O.reduce_sum(np.abs(X).astype(np.float64), axes, keepdims)   # every element, not only the norm
        assert (np.abs(Y - expected) <= 5e-6 * abs_sum).all()
    else:
        assert np.array_equal(expected.astype(np.float32), Y)


def test_reduce_max_min_propagate_nan():
    X = np.random.default_rng(18).normal(size=(6, 50)).astype(np.float32)
    X[2, 17] = np.nan
    for op, oracle in (("ReduceMax", O.reduce_max), ("ReduceMin", O.reduce_min)):
        for axes in ([1], [0]):
            expected = oracle(X, axes, 0)
            Y = np.zeros(expected.shape, np.float32)
            getattr(donnx, "ONNX" + op)(data=X, reduced=Y, axes=axes, keepdims=0)
            assert np.array_equal(expected, Y, equal_nan=True), (op, axes)


@pytest.mark.parametrize("shape, axis", [((8, 12, 128, 128), -1), ((5, 48), -1), ((3, 1000), 1), ((2, 5000), -1),
                                         ((3, 30), -1), ((3, 17, 5, 9), 1), ((4, 6, 48), 0), ((3, 1), -1)])
def test_log_softmax(shape, axis):
    """PureLogSoftmax (pure_implementations.py:594-616); also exp(result) must sum to one along the axis."""
    X = np.random.default_rng(19).normal(scale=4, size=shape).astype(np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXLogSoftmax(input=X, output=Y, axis=axis)
    expected = O.log_softmax(X.astype(np.float64), axis=axis)
    assert np.allclose(Y, expected, rtol=1e-5, atol=2e-6), np.abs(Y - expected).max()
    assert np.allclose(np.exp(Y.astype(np.float64)).sum(axis), 1.0, atol=1e-4)
    assert np.allclose(Y, torch.nn.functional.log_softmax(torch.from_numpy(X), dim=axis).numpy(), rtol=1e-5, atol=2e-6)


def test_log_softmax_large_values():
    X = np.array([[1000.0, 999.0, -1000.0, 0.0]] * 3, np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXLogSoftmax(input=X, output=Y, axis=1)
    assert np.isfinite(Y).all() and np.allclose(Y, O.log_softmax(X.astype(np.float64), axis=1), rtol=1e-6)


@pytest.mark.parametrize("count", [1, 2, 3, 4])
@pytest.mark.parametrize("shape", [(8, 16, 768), (7, ), (3, 5)])
def test_sum(count, shape):
    """PureSum (pure_implementations.py:529-591): inputs of one shape, added left to right -- bit-exact."""
    rng = np.random.default_rng(20)
    xs = [rng.normal(size=shape).astype(np.float32) for _ in range(count)]
    Y = np.zeros(shape, np.float32)
    donnx.ONNXSum(**{f"data_0__{i}": x for i, x in enumerate(xs)}, sum=Y)
    assert np.array_equal(O.sum_(*xs), Y)


@pytest.mark.parametrize("src, dst", [(np.float32, np.int32), (np.float32, np.int64), (np.int64, np.float32),
                                      (np.int32, np.int64), (np.int64, np.int32), (np.float32, np.float64),
                                      (np.float64, np.float32), (np.float32, np.bool_), (np.int8, np.float32),
                                      (np.uint8, np.int32), (np.float32, np.int8), (np.bool_, np.float32),
                                      (np.float32, np.float32)])
@pytest.mark.parametrize("n", [1, 1000, 70001])
def test_cast(src, dst, n):
    """PureCast (pure_implementations.py:382-430): the C conversion, element by element, exact."""
    rng = np.random.default_rng(23)
    X = (rng.normal(scale=40, size=n) * (rng.random(n) > 0.2)).astype(src)       # zeros included, for bool
    Y = np.zeros(n, dst)
    donnx.ONNXCast(input=X, output=Y, to=proto.np_dtype_to_tensor_dtype(np.dtype(dst)))
    assert Y.dtype == np.dtype(dst) and np.array_equal(O.cast(X, dst), Y)


@pytest.mark.parametrize("shape, starts, ends, axes, steps", [
    ((2, ), [0], [1], [0], None),                                    # the reference's slice.onnx
    ((512, 768), [0, 0], [256, 2 ** 63 - 1], None, None),            # the reference's reshape.onnx
    ((20, 10, 6), [5], [2 ** 63 - 1], [0], [1]),                     # PureSlice's own case: axis 0, step 1, "to the end"
    ((20, 10, 6), [1, 2], [18, -1], [0, 2], [3, 2]),
    ((4, 9, 33), [-2, 30], [100, 3], [1, 2], [1, -4]),
    ((7, 8), [6], [-100], [0], [-1]),
    ((7, 8), [3], [3], [1], [1]),                                    # empty result
    ((3, 130, 70), [1, 2], [129, 69], [-2, -1], [1, 1])])
def test_slice(shape, starts, ends, axes, steps):
    X = np.random.default_rng(24).normal(size=shape).astype(np.float32)
    expected = O.slice_(X, starts, ends, axes, steps)
    Y = np.full(expected.shape, np.nan, np.float32)
    as_i64 = lambda v: None if v is None else np.array(v, dtype=np.int64)
    kwargs = {k: as_i64(v) for k, v in (("starts", starts), ("ends", ends), ("axes", axes), ("steps", steps)) if v is not None}
    donnx.ONNXSlice(data=X, output=Y, **kwargs)
    assert np.array_equal(expected, Y)
    Xi = np.arange(int(np.prod(shape)), dtype=np.int32).reshape(shape)          # any 4-byte element type
    Yi = np.zeros(expected.shape, np.int32)
    donnx.ONNXSlice(data=Xi, output=Yi, **kwargs)
    assert np.array_equal(O.slice_(Xi, starts, ends, axes, steps), Yi)


@pytest.mark.parametrize("equation, shapes", [
    ("bij ,jk -> bik", [(5, 4, 3), (3, 2)]),                 # tests/pure_expansions/test_expansions.py:456-473 (there in fp64)
    ("ik,kj->ij", [(33, 20), (20, 48)]),
    ("bhqd,bhkd->bhqk", [(2, 3, 16, 8), (2, 3, 20, 8)]),     # Q K^T
    ("bhqk,bhkd->bhqd", [(2, 3, 16, 20), (2, 3, 20, 8)]),    # P V
    ("bqhd,bkhd->bhqk", [(2, 16, 3, 8), (2, 20, 3, 8)]),     # heads not split out beforehand
    ("bik,jk->bij", [(4, 10, 12), (7, 12)]),                 # Linear: x W^T
    ("ij,bjk->bik", [(6, 5), (3, 5, 8)]),                    # shared left operand
    ("bij,bjk->bki", [(3, 6, 5), (3, 5, 8)]),                # transposed result: the inputs change roles
    ("abc,cd->abd", [(2, 3, 4), (4, 4)]),
    ("ijk,jkl->il", [(6, 4, 5), (4, 5, 7)]),                 # two contracted letters walked as one axis
    ("i,j->ij", [(9, ), (12, )]),                            # outer product (K = 1)
    ("bi,bi->b", [(6, 40), (6, 40)])])                       # batched dot product (M = N = 1)
def test_einsum(equation, shapes):
    rng = np.random.default_rng(25)
    xs = [rng.normal(size=s).astype(np.float32) for s in shapes]
    expected = O.einsum(equation, *[x.astype(np.float64) for x in xs])
    Y = np.zeros(expected.shape, np.float32)
    donnx.ONNXEinsum(Inputs__0=xs[0], Inputs__1=xs[1], Output=Y, equation=equation)
    assert rel_err(expected, Y) < FP32_REL_TOL


@pytest.mark.parametrize("equation, shapes", [("ii->i", [(4, 4)]), ("ij,jk,kl->il", [(2, 3), (3, 4), (4, 5)]),
                                              ("ij,jk->i", [(2, 3), (3, 4)]), ("...ij,jk->...ik", [(2, 2, 3), (3, 4)]),
                                              ("ijk,kjl->il", [(6, 4, 5), (5, 4, 7)])])
def test_einsum_refuses_what_one_gemm_cannot_do(equation, shapes):
    xs = [np.zeros(s, np.float32) for s in shapes]
    out_shape = np.einsum(equation, *xs).shape
    with pytest.raises(donnx.ExpansionRefused):
        donnx.ONNXEinsum(**{f"Inputs__{i}": x for i, x in enumerate(xs)}, Output=np.zeros(out_shape, np.float32), equation=equation)


@pytest.mark.parametrize("shape, kernel, strides, pads, dil", [
    ((5, 3, 10, 10), (2, 2), (2, 2), None, None),                       # LeNet-style pooling
    ((2, 64, 112, 112), (3, 3), (2, 2), (1, 1, 1, 1), None),             # ResNet stem
    ((1, 2, 9, 11), (3, 2), (1, 2), (1, 0, 2, 1), None), ((3, 4, 17, 13), (2, 3), (1, 1), (0, 1, 0, 1), (2, 2)),
    ((2, 3, 7, 7), (7, 7), None, None, None),
    # large enough for the variant that stages bands of rows through LDS: rows that are not a multiple of 16 bytes,
    # a window with different extents and dilation, 2 x 2 / 2, and a plane too wide for the staging buffer
    ((3, 40, 61, 47), (3, 2), (2, 1), (1, 0, 2, 1), (1, 2)), ((2, 48, 56, 56), (2, 2), (2, 2), None, None),
    ((4, 30, 33, 36), (3, 3), (1, 1), (1, 1, 1, 1), None), ((1, 6, 20, 3000), (3, 3), (2, 2), (1, 1, 1, 1), None)])
def test_maxpool(shape, kernel, strides, pads, dil):
    """PureMaxPool2D (img_op_implementations.py:28-161), plus pads / dilations: exact."""
    X = np.random.default_rng(27).normal(size=shape).astype(np.float32)
    expected = O.maxpool2d(X, kernel, strides or (1, 1), pads or (0, 0, 0, 0), dil or (1, 1))
    Y = np.zeros(expected.shape, np.float32)
    attrs = {k: list(v) for k, v in (("strides", strides), ("pads", pads), ("dilations", dil)) if v is not None}
    donnx.ONNXMaxPool(X=X, Y=Y, kernel_shape=list(kernel), **attrs)
    assert np.array_equal(expected, Y)


def test_maxpool_nan_and_refusals():
    X = np.random.default_rng(28).normal(size=(1, 1, 6, 6)).astype(np.float32)
    X[0, 0, 2, 3] = np.nan
    Y = np.zeros((1, 1, 3, 3), np.float32)
    donnx.ONNXMaxPool(X=X, Y=Y, kernel_shape=[2, 2], strides=[2, 2])
    assert np.array_equal(O.maxpool2d(X, (2, 2), (2, 2)), Y, equal_nan=True) and np.isnan(Y).sum() == 1
    with pytest.raises(donnx.ExpansionRefused):
        donnx.ONNXMaxPool(X=X, Y=np.zeros((1, 1, 3, 3), np.float32), kernel_shape=[2, 2], strides=[2, 2], ceil_mode=1)


@pytest.mark.parametrize("shape", [(32, 64, 56, 56), (2, 3, 7, 5), (4, 16, 1, 1), (1, 5, 33)])
def test_global_average_pool_and_batch_normalization(shape):
    rng = np.random.default_rng(29)
    X = rng.normal(1.0, 2.0, size=shape).astype(np.float32)
    Y = np.zeros(shape[:2] + (1, ) * (len(shape) - 2), np.float32)
    donnx.ONNXGlobalAveragePool(X=X, Y=Y)
    assert rel_err(O.global_average_pool(X.astype(np.float64)), Y) < FP32_REL_TOL
    C = shape[1]
    scale, b, mean = (rng.normal(size=C).astype(np.float32) for _ in range(3))
    var = rng.uniform(0.5, 2.0, size=C).astype(np.float32)
    Z = np.zeros_like(X)
    donnx.ONNXBatchNormalization(X=X, scale=scale, B=b, in_mean=mean, in_var=var, Y=Z, epsilon=1e-3)
    expected = O.batch_normalization(X, scale, b, mean, var, 1e-3)
    assert np.allclose(Z, expected, rtol=1e-5, atol=1e-5) and rel_err(expected, Z) < 1e-6


def _single_node_sdfg(sdfg_name, node, inputs, out_conn, out_shape, out_dtype=None):
    """The hand-built one-node SDFG of the reference's expansion tests: arrays, one state, the node, its edges."""
    sdfg = dace.SDFG(sdfg_name)
    state = sdfg.add_state()
    state.add_node(node)
    for conn, (name, value) in inputs.items():
        sdfg.add_array(name, list(value.shape), dace.typeclass_of(value.dtype))
        state.add_edge(state.add_access(name), None, node, conn, sdfg.make_array_memlet(name))
    sdfg.add_array("__return", list(out_shape), out_dtype or dace.float32)
    state.add_edge(node, out_conn, state.add_access("__return"), None, sdfg.make_array_memlet("__return"))
    sdfg.expand_library_nodes()
    assert_expanded_to_kernels(sdfg)
    return sdfg


@pytest.mark.parametrize("reduce_type, keepdims, axes", [("Sum", True, [0]), ("Sum", False, [-1]), ("Sum", True, [0, -1]),
                                                         ("Max", False, [0, -1]), ("Max", True, [0]), ("Max", True, [-1]),
                                                         ("Mean", True, [-1]), ("Mean", True, [0, -1]), ("Mean", False, [0]),
                                                         ("Min", False, [0, -1]), ("Min", True, [1])])
def test_reduce(keepdims, reduce_type, axes, sdfg_name):
    # tests/pure_expansions/test_expansions.py:176-230 (its grid, including the non-adjacent axes [0, -1]), plus Min
    X = np.random.default_rng(32).normal(scale=10, size=(2, 4, 10)).astype(np.float32)
    numpy_result = getattr(np, reduce_type.lower())(X.copy(), axis=tuple(axes), keepdims=keepdims)
    op_node = getattr(donnx, "ONNXReduce" + reduce_type)("reduce")
    op_node.axes = axes
    op_node.keepdims = 1 if keepdims else 0
    sdfg = _single_node_sdfg(sdfg_name, op_node, {"data": ("X", X)}, "reduced", numpy_result.shape)
    result = sdfg(X=X)
    assert np.allclose(numpy_result, result, rtol=1e-5, atol=1e-5)


def test_reduce_scalar(sdfg_name):
    # tests/pure_expansions/test_expansions.py:233-270: no axes attribute, keepdims 0 -> every axis, one value
    X = np.random.default_rng(33).normal(scale=10, size=(2, 4, 10)).astype(np.float32)
    op_node = donnx.ONNXReduceMean("mean")
    op_node.keepdims = 0
    sdfg = _single_node_sdfg(sdfg_name, op_node, {"data": ("X", X)}, "reduced", ())
    assert np.allclose(np.mean(X), sdfg(X=X))


@pytest.mark.parametrize("shape, axes", [((6, 5, 7, 3), [0, 2]), ((6, 5, 7, 3), [1, 3]), ((3, 130, 4, 70), [1, 3]),
                                         ((2, 3, 4, 5, 6), [0, 2, 4])])
@pytest.mark.parametrize("op", ["ReduceSum", "ReduceMax", "ReduceMin", "ReduceMean"])
def test_reduce_non_adjacent_axes(op, shape, axes):
    X = np.random.default_rng(34).normal(1.0, 2.0, size=shape).astype(np.float32)
    oracle = {"ReduceSum": O.reduce_sum, "ReduceMax": O.reduce_max, "ReduceMin": O.reduce_min, "ReduceMean": O.reduce_mean}[op]
    for keepdims in (0, 1):
        expected = oracle(X.astype(np.float64), axes, keepdims)
        Y = np.zeros(expected.shape, np.float32)
        getattr(donnx, "ONNX" + op)(data=X, reduced=Y, axes=axes, keepdims=keepdims)
        if op in ("ReduceMax", "ReduceMin"):
            assert np.array_equal(expected.astype(np.float32), Y)
        else:
            assert np.allclose(Y, expected, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("src, dst", [(np.int32, np.float32), (np.float32, np.int32), (np.float32, np.int64)])
def test_cast_reference_cases(src, dst, sdfg_name):
    # tests/pure_expansions/test_expansions.py:78-174: int -> float, float -> int, float -> long on a [2, 4, 10] array
    X = np.random.default_rng(35).normal(scale=10, size=(2, 4, 10)).astype(src)
    op_node = donnx.ONNXCast("Cast", to=proto.np_dtype_to_tensor_dtype(np.dtype(dst)))   # `to` is a required attribute
    sdfg = _single_node_sdfg(sdfg_name, op_node, {"input": ("X", X)}, "output", X.shape, dace.typeclass_of(np.dtype(dst)))
    result = sdfg(X=X)
    assert result.dtype == np.dtype(dst) and np.array_equal(X.astype(dst), result)


def test_cast_scalar():
    # tests/pure_expansions/test_expansions.py:61-75: a float64 scalar to float32
    out = np.zeros((), np.float32)
    donnx.ONNXCast(input=np.array(2.0, np.float64), output=out, to=proto.np_dtype_to_tensor_dtype(np.dtype(np.float32)))
    assert out == 2


@pytest.mark.parametrize("shape", [(2, 3), (1, ), ()])
def test_sum_arrays(shape):
    # tests/pure_expansions/test_expansions.py:500-530: three inputs of one shape, also [1] and scalars
    rng = np.random.default_rng(36)
    inputs = [np.asarray(rng.normal(size=shape), dtype=np.float32) for _ in range(3)]
    result = np.zeros(shape, np.float32)
    donnx.ONNXSum(data_0__0=inputs[0], data_0__1=inputs[1], data_0__2=inputs[2], sum=result)
    assert np.allclose(result, (inputs[0] + inputs[1]) + inputs[2])


def test_reshape_then_add():
    # tests/pure_expansions/test_expansions.py:477-497: Reshape whose target is a run-time input; the result's shape
    # is the declared one
    inp, bias = np.arange(9).astype(np.float32), np.arange(3).astype(np.float32)
    reshaped, out = np.zeros((3, 3), np.float32), np.zeros((3, 3), np.float32)
    donnx.ONNXReshape(data=inp, shape=np.array([3, 3]).astype(np.int64), reshaped=reshaped)
    donnx.ONNXAdd(A=reshaped, B=bias, C=out)
    assert np.allclose(out, inp.reshape(3, 3) + bias)


def test_reciprocal_and_logsoftmax_reference_cases(sdfg_name):
    # tests/pure_expansions/test_expansions.py:384-453
    X = np.random.default_rng(37).normal(scale=10, size=(2, 4, 10)).astype(np.float32)
    for axis in (0, 1, 2, -1):
        Y = np.zeros_like(X)
        donnx.ONNXLogSoftmax(input=X, output=Y, axis=axis)
        assert np.linalg.norm(torch.nn.functional.log_softmax(torch.from_numpy(X), dim=axis).numpy() - Y) < 1e-5
    sdfg = _single_node_sdfg(sdfg_name, donnx.ONNXReciprocal("reciprocal"), {"X": ("X", X)}, "Y", X.shape)
    assert np.allclose(1 / X, sdfg(X=X))


@pytest.mark.parametrize("shape, axes", [((1, ), None), ((1, ), [0]), ((3, 1, 5, 1), [1, 3]), ((3, 1, 5, 1), [-1]), ((3, 1, 5, 1), None)])
def test_squeeze_then_unsqueeze(shape, axes, sdfg_name):
    # tests/test_input_outputs.py:43-95 of the reference: Squeeze an array (there: of one element, to a scalar) and
    # Unsqueeze it back, as views of the same storage
    X = np.random.default_rng(38).random(shape).astype(np.float32)
    squeezed_shape = np.squeeze(X, axis=tuple(axes) if axes is not None else None).shape
    back_axes = sorted(a % len(shape) for a in axes) if axes is not None else [i for i, d in enumerate(shape) if d == 1]
    sdfg = dace.SDFG(sdfg_name)
    sdfg.add_array("X_arr", list(shape), dace.float32)
    sdfg.add_transient("squeezed", list(squeezed_shape), dace.float32)
    sdfg.add_array("__return", list(shape), dace.float32)
    state = sdfg.add_state()
    sq = donnx.ONNXSqueeze("Squeeze", **({"axes": axes} if axes is not None else {}))
    unsq = donnx.ONNXUnsqueeze("Unsqueeze", axes=back_axes)
    mid = state.add_access("squeezed")
    state.add_node(sq)
    state.add_node(unsq)
    state.add_edge(state.add_access("X_arr"), None, sq, "data", sdfg.make_array_memlet("X_arr"))
    state.add_edge(sq, "squeezed", mid, None, sdfg.make_array_memlet("squeezed"))
    state.add_edge(mid, None, unsq, "data", sdfg.make_array_memlet("squeezed"))
    state.add_edge(unsq, "expanded", state.add_access("__return"), None, sdfg.make_array_memlet("__return"))
    sdfg.expand_library_nodes()
    assert_expanded_to_kernels(sdfg)
    assert np.array_equal(sdfg(X_arr=X), X)


def test_bn_standalone():
    # tests/test_shared_input_output.py:17-41 of the reference: `mean` / `var` name an input and an output of the ONNX
    # operator, so the connectors are in_mean / in_var (and out_mean / out_var)
    X, scale, B, mean = torch.randn(8, 3, 32, 32), torch.randn(3), torch.randn(3), torch.randn(3)
    var = torch.rand(3) + 0.5
    Y = np.zeros((8, 3, 32, 32), np.float32)
    donnx.ONNXBatchNormalization(X=X.numpy(), scale=scale.numpy(), B=B.numpy(), in_mean=mean.numpy(), in_var=var.numpy(), Y=Y)
    pt_result = torch.nn.functional.batch_norm(X, mean, var, scale, B)
    assert np.allclose(pt_result.numpy(), Y, rtol=1e-5, atol=1e-4)
    with pytest.raises(TypeError, match="Unknown arguments"):
        donnx.ONNXBatchNormalization(X=X.numpy(), scale=scale.numpy(), B=B.numpy(), mean=mean.numpy(), var=var.numpy(), Y=Y)


def test_pow():
    rng = np.random.default_rng(16)
    X = rng.normal(size=(8, 16, 64)).astype(np.float32)
    Z = np.zeros_like(X)
    donnx.ONNXPow(X=X, Y=np.array(2.0, np.float32), Z=Z)
    assert np.array_equal(O.pow(X, 2.0), Z)                 # the exponent of the exported LayerNorm: exact
    P = np.abs(X) + 0.25
    E = rng.uniform(-2, 3, size=(64, )).astype(np.float32)  # broadcast exponent
    donnx.ONNXPow(X=P, Y=E, Z=Z)
    assert rel_err(O.pow(P.astype(np.float64), E.astype(np.float64)), Z) < FP32_REL_TOL


# ----------------------------------------------------------------------------- data movement
@pytest.mark.parametrize("shape, perm", [((8, 16, 12, 64), (0, 2, 1, 3)), ((2, 12, 16, 64), (0, 1, 3, 2)),
                                         ((5, 7), None), ((3, 4, 5), (2, 0, 1)), ((70, 130), (1, 0)), ((6, ), (0, ))])
def test_transpose(shape, perm):
    X = np.random.default_rng(11).normal(size=shape).astype(np.float32)
    expected = O.transpose(X, perm)
    Y = np.zeros(expected.shape, np.float32)
    kwargs = {} if perm is None else {"perm": list(perm)}
    donnx.ONNXTranspose(data=X, transposed=Y, **kwargs)
    assert np.array_equal(expected, Y)


def test_reshape_is_a_view_inside_a_graph():
    # Reshape between two kernels moves no data: the SDFG has two kernel calls and one alias
    sdfg = dace.SDFG("reshape_chain")
    sdfg.add_array("X", [4, 6], dace.float32)
    sdfg.add_array("shape", [3], dace.int64)
    sdfg.add_transient("r", [4, 6], dace.float32)
    sdfg.add_transient("v", [2, 3, 4], dace.float32)
    sdfg.add_array("__return", [2, 3, 4], dace.float32)
    st = sdfg.add_state()
    relu, resh, gelu = donnx.ONNXRelu("relu"), donnx.ONNXReshape("reshape"), donnx.ONNXGelu("gelu")
    ar, av = st.add_access("r"), st.add_access("v")
    st.add_edge(st.add_read("X"), None, relu, "X", sdfg.make_array_memlet("X"))
    st.add_edge(relu, "Y", ar, None, sdfg.make_array_memlet("r"))
    st.add_edge(ar, None, resh, "data", sdfg.make_array_memlet("r"))
    st.add_edge(st.add_read("shape"), None, resh, "shape", sdfg.make_array_memlet("shape"))
    st.add_edge(resh, "reshaped", av, None, sdfg.make_array_memlet("v"))
    st.add_edge(av, None, gelu, "X", sdfg.make_array_memlet("v"))
    st.add_edge(gelu, "Y", st.add_write("__return"), None, sdfg.make_array_memlet("__return"))
    utils.expand_onnx_nodes(sdfg)
    kinds = [type(n).__name__ for n, _ in sdfg.all_nodes_recursive() if isinstance(n, (dace.KernelCall, dace.AliasNode))]
    assert sorted(kinds) == ["AliasNode", "KernelCall", "KernelCall"]
    X = np.random.default_rng(12).normal(size=(4, 6)).astype(np.float32)
    out = sdfg(X=X, shape=np.array([2, 3, 4], np.int64))
    assert rel_err(O.gelu(O.relu(X)).reshape(2, 3, 4), out) < FP32_REL_TOL


# ----------------------------------------------------------------------------- MatMulInteger
@pytest.mark.parametrize("M, N, K, za, zb", [(128, 128, 64, 0, 0), (128, 128, 64, 3, -2), (512, 384, 768, 3, -2),
                                             (100, 52, 37, 5, 7), (130, 260, 48, -128, 127), (1, 1, 1, 1, 1),
                                             (33, 2, 16, 0, 9), (7, 129, 1000, -7, 0),
                                             # K % 64 == 0 and N % 16 == 0: the pipelined kernel, ragged M and N tiles
                                             (200, 144, 256, 3, -2), (1, 16, 128, -128, 127), (257, 400, 640, 0, 11),
                                             (129, 112, 1152, -9, 0), (130, 272, 64, 5, 5),
                                             (128, 128, 128, 0, 0), (200, 132, 256, 3, -2), (1, 4, 128, -128, 127),
                                             (257, 388, 640, 0, 11), (129, 124, 1152, -9, 0), (384, 256, 384, 1, 1)])
def test_matmul_integer_bit_exact(M, N, K, za, zb):
    rng = np.random.default_rng(13)
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    Y = np.zeros((M, N), np.int32)
    donnx.ONNXMatMulInteger(A=A, B=B, a_zero_point=np.array(za, np.int8), b_zero_point=np.array(zb, np.int8), Y=Y)
    assert np.array_equal(O.matmul_integer(A, B, za, zb), Y)


def test_matmul_integer_without_zero_points_and_extremes():
    A = np.full((64, 768), -128, np.int8)
    B = np.full((768, 32), -128, np.int8)
    Y = np.zeros((64, 32), np.int32)
    donnx.ONNXMatMulInteger(A=A, B=B, Y=Y)
    assert np.all(Y == 768 * 128 * 128)
    donnx.ONNXMatMulInteger(A=A, B=B, a_zero_point=np.array([127], np.int8), b_zero_point=np.array([127], np.int8), Y=Y)
    assert np.all(Y == 768 * 255 * 255)


@pytest.mark.parametrize("a_dt, b_dt", [(np.uint8, np.int8), (np.int8, np.uint8), (np.uint8, np.uint8)])
@pytest.mark.parametrize("M, N, K", [(256, 256, 128), (200, 144, 192), (100, 52, 37), (384, 256, 64), (1, 16, 64)])
def test_matmul_integer_unsigned_operands_bit_exact(a_dt, b_dt, M, N, K):
    """uint8 operands (ONNX MatMulInteger T1 / T2, the node class of onnx_op.py:623-640): scalar zero points of the
    operand's type, no zero points, against the integer formula. Parity unpinned against the reference itself,
    which runs the node only inside ONNX Runtime."""
    rng = np.random.default_rng(31)
    A = rng.integers(0, 256, size=(M, K)).astype(a_dt) if a_dt == np.uint8 else rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(0, 256, size=(K, N)).astype(b_dt) if b_dt == np.uint8 else rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    za, zb = np.array(131 if a_dt == np.uint8 else -3, a_dt), np.array(250 if b_dt == np.uint8 else 7, b_dt)
    Y = np.zeros((M, N), np.int32)
    donnx.ONNXMatMulInteger(A=A, B=B, a_zero_point=za, b_zero_point=zb, Y=Y)
    assert np.array_equal(O.matmul_integer(A, B, za, zb), Y)
    donnx.ONNXMatMulInteger(A=A, B=B, Y=Y)
    assert np.array_equal(O.matmul_integer(A, B), Y)
    donnx.ONNXMatMulInteger(A=A, B=B, b_zero_point=zb, Y=Y)
    assert np.array_equal(O.matmul_integer(A, B, 0, zb), Y)


@pytest.mark.parametrize("M, N, K", [(256, 256, 128), (130, 80, 64), (77, 36, 50)])
def test_matmul_integer_zero_point_per_row_and_column(M, N, K):
    rng = np.random.default_rng(32)
    A = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    za = rng.integers(0, 256, size=M).astype(np.uint8)
    zb = rng.integers(-128, 128, size=N, dtype=np.int8)
    Y = np.zeros((M, N), np.int32)
    donnx.ONNXMatMulInteger(A=A, B=B, a_zero_point=za, b_zero_point=zb, Y=Y)
    assert np.array_equal(O.matmul_integer(A, B, za, zb), Y)
    donnx.ONNXMatMulInteger(A=A, B=B, a_zero_point=za, Y=Y)
    assert np.array_equal(O.matmul_integer(A, B, za, 0), Y)


def test_matmul_integer_stack_of_matrices():
    rng = np.random.default_rng(33)
    A = rng.integers(-128, 128, size=(3, 64, 128), dtype=np.int8)
    B = rng.integers(-128, 128, size=(128, 48), dtype=np.int8)
    za = rng.integers(-128, 128, size=(3, 64, 1), dtype=np.int8)
    Y = np.zeros((3, 64, 48), np.int32)
    donnx.ONNXMatMulInteger(A=A, B=B, a_zero_point=za, b_zero_point=np.array(-2, np.int8), Y=Y)
    assert np.array_equal(O.matmul_integer(A, B, za, -2), Y)


def test_matmul_integer_several_tiles_per_workgroup():
    """More 128 x 128 tiles than resident workgroups: a workgroup stores one tile while it multiplies the next."""
    rng = np.random.default_rng(34)
    M, N, K = 4096, 4096, 128
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    Y = np.zeros((M, N), np.int32)
    donnx.ONNXMatMulInteger(A=A, B=B, a_zero_point=np.array(3, np.int8), b_zero_point=np.array(-2, np.int8), Y=Y)
    ref = (A.astype(np.int32) - 3) @ (B.astype(np.int32) + 2)
    assert np.array_equal(ref, Y)


# ----------------------------------------------------------------------------- edge cases
def test_empty_inputs():
    X = np.zeros((0, 128), np.float32)
    Y = np.zeros((0, 128), np.float32)
    donnx.ONNXSoftmax(input=X, output=Y, axis=-1)
    donnx.ONNXRelu(X=X, Y=Y)
    A, B, C = np.zeros((0, 8), np.float32), np.zeros((8, 4), np.float32), np.zeros((0, 4), np.float32)
    donnx.ONNXMatMul(A=A, B=B, Y=C)
    # K == 0: the product is all zeros
    A, B, C = np.zeros((3, 0), np.float32), np.zeros((0, 4), np.float32), np.ones((3, 4), np.float32)
    donnx.ONNXMatMul(A=A, B=B, Y=C)
    assert np.all(C == 0)


def test_torch_tensors_stay_on_device():
    x = torch.randn(64, 128, device="cuda")
    y = torch.empty_like(x)
    donnx.ONNXSoftmax(input=x, output=y, axis=-1)
    torch.cuda.synchronize()
    assert rel_err(O.softmax(x.cpu().numpy()), y.cpu().numpy()) < FP32_REL_TOL


# ----------------------------------------------------------------------------- elementwise programs
def _ins(op, dst, a, b=0):
    return op | (dst << 8) | (a << 16) | (b << 24)


def _opnd(kind, idx):
    return (kind << 6) | idx


@pytest.mark.parametrize("shape", [(6, 40, 768), (5, 7, 9), (1, 4), (3, 1)])
def test_eltwise_program_c_abi(shape):
    # y = gelu((t0 * 0.5 + v0) / t1) - relu(v1 * t0): tensors, vectors along the last axis, immediates, registers
    R, TN, VC, IM = _lib.PROGRAM_REG, _lib.PROGRAM_TENSOR, _lib.PROGRAM_VECTOR, _lib.PROGRAM_IMMEDIATE
    rng = np.random.default_rng(sum(shape))
    t0 = rng.normal(size=shape).astype(np.float32)
    t1 = (rng.random(size=shape) + 0.5).astype(np.float32)
    v0, v1 = rng.normal(size=shape[-1]).astype(np.float32), rng.normal(size=shape[-1]).astype(np.float32)
    program = [_ins(_lib.OP_MUL, 0, _opnd(TN, 0), _opnd(IM, 0)),
               _ins(_lib.OP_ADD, 0, _opnd(R, 0), _opnd(VC, 0)),
               _ins(_lib.OP_DIV, 1, _opnd(R, 0), _opnd(TN, 1)),
               _ins(_lib.OP_GELU, 1, _opnd(R, 1)),
               _ins(_lib.OP_MUL, 2, _opnd(VC, 1), _opnd(TN, 0)),
               _ins(_lib.OP_RELU, 2, _opnd(R, 2)),
               _ins(_lib.OP_SUB, 0, _opnd(R, 1), _opnd(R, 2))]
    expected = O.sub(O.gelu(O.div(O.add(O.mul(t0, np.float32(0.5)), v0), t1)), O.relu(O.mul(v1, t0)))
    dt = [torch.from_numpy(a).cuda() for a in (t0, t1, v0, v1)]
    y = torch.full(shape, float("nan"), device="cuda")
    lib = _lib.library()
    call = lambda prog, n_t=2, n_v=2, n_imm=1: lib.mi355x_eltwise_program_f32(
        _lib.pointer_array([dt[0].data_ptr(), dt[1].data_ptr()]), n_t, _lib.pointer_array([dt[2].data_ptr(), dt[3].data_ptr()]),
        n_v, y.data_ptr(), y.numel(), shape[-1], _lib.u32_array(prog), len(prog), _lib.f32_array([0.5]), n_imm,
        _lib.current_stream())
    _lib.check(call(program), "mi355x_eltwise_program_f32")
    assert rel_err(expected, y.cpu().numpy()) < FP32_REL_TOL
    # malformed programs are refused before anything is launched: a register read before it is written, an input
    # that does not exist, an unknown opcode
    assert call([_ins(_lib.OP_ADD, 0, _opnd(R, 3), _opnd(TN, 0))]) == 1
    assert "does not exist" in lib.mi355x_last_error().decode()
    assert call([_ins(_lib.OP_ADD, 0, _opnd(TN, 0), _opnd(VC, 1))], n_v=1) == 1
    assert call([_ins(9, 0, _opnd(TN, 0), _opnd(TN, 0))]) == 1
    assert call(program * 3) == 1     # 21 instructions

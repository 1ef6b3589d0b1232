"""Pins the oracle (CPU restatement of the reference's expansions).

The reference's tests hold no golden vectors: each recomputes its expectation
with numpy / PyTorch (tests/pure_expansions/test_expansions.py:29,349;
test_conv_expansion.py:30-35). The same comparators are used here, plus the
committed fixtures (PyTorch float64), closed forms, invariants and brute force,
chosen so that a dropped term, a wrong sign/index or a transposed operand fails.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import pure_ops as O
from conftest import rel_err

TOL = 2e-6  # oracle is fp32 numpy; comparators are float64


# ----------------------------------------------------------------------------- golden fixtures
def test_golden_conv_config1(golden):
    y = O.conv2d(golden["conv1_X"], golden["conv1_W"], strides=(2, 2))
    assert y.shape == (5, 16, 4, 4)
    assert rel_err(golden["conv1_Y"], y) < TOL


def test_golden_conv_pads_dilation_bias_relu(golden):
    y = O.relu(O.conv2d(golden["conv2_X"], golden["conv2_W"], golden["conv2_B"], strides=(2, 1),
                        pads=(1, 2, 0, 1), dilations=(1, 2)))
    assert rel_err(golden["conv2_Y"], y) < TOL


def test_golden_softmax_layernorm_gelu(golden):
    assert rel_err(golden["softmax_Y"], O.softmax(golden["softmax_X"], axis=-1)) < TOL
    assert rel_err(golden["ln_Y"], O.layer_normalization(golden["ln_X"], golden["ln_gamma"], golden["ln_beta"],
                                                         axis=-1, epsilon=1e-12)) < TOL
    assert rel_err(golden["gelu_Y"], O.gelu(golden["gelu_X"])) < TOL


def test_golden_matmul_gemm(golden):
    assert rel_err(golden["matmul_Y"], O.matmul(golden["matmul_A"], golden["matmul_B"])) < TOL
    assert rel_err(golden["gemm_Y"], O.gemm(golden["gemm_A"], golden["gemm_B"], golden["gemm_C"], transB=1)) < TOL


def test_golden_matmul_integer(golden):
    y = O.matmul_integer(golden["mmi_A"], golden["mmi_B"], 3, -2)
    assert y.dtype == np.int32 and np.array_equal(y, golden["mmi_Y"])


def test_golden_bert_layer(golden):
    hidden, heads, ffn, bsz, seq = (int(v) for v in golden["bert_meta"])
    w = {k[len("bert_"):]: golden[k] for k in golden.files if k.startswith("bert_") and k not in
         ("bert_x", "bert_y", "bert_meta")}
    y = O.bert_layer(golden["bert_x"], w, heads=heads)
    assert y.shape == (bsz, seq, hidden)
    assert rel_err(golden["bert_y"], y) < 5e-6


# ----------------------------------------------------------------------------- matmul / gemm
def test_matmul_einsum_strings():
    # the strings PureMatMul produces (pure_implementations.py:151-210)
    assert O.matmul_einsum_string(2, 2) == "ik,kj->ij"
    assert O.matmul_einsum_string(3, 2) == "aik,kj->aij"
    assert O.matmul_einsum_string(4, 4) == "baik,bakj->baij"
    assert O.matmul_einsum_string(2, 3) == "ik,akj->aij"
    with pytest.raises(ValueError):
        O.matmul_einsum_string(1, 2)


@pytest.mark.parametrize("a_shape, b_shape", [([2, 4], [4, 3]), ([8, 12, 16, 8], [8, 12, 8, 16]),
                                              ([3, 5, 7], [7, 2]), ([5, 7], [3, 7, 2]), ([2, 1, 4, 6], [3, 6, 5])])
def test_matmul_vs_numpy_float64(a_shape, b_shape):
    rng = np.random.default_rng(0)
    A = rng.random(a_shape).astype(np.float32)
    B = rng.random(b_shape).astype(np.float32)
    assert rel_err(A.astype(np.float64) @ B.astype(np.float64), O.matmul(A, B)) < TOL


def test_matmul_bruteforce_small():
    rng = np.random.default_rng(1)
    A = rng.normal(size=(5, 7)).astype(np.float32)
    B = rng.normal(size=(7, 6)).astype(np.float32)
    ref = np.zeros((5, 6))
    for i in range(5):
        for j in range(6):
            for k in range(7):
                ref[i, j] += float(A[i, k]) * float(B[k, j])
    assert rel_err(ref, O.matmul(A, B)) < TOL
    # a transposed operand must fail this check
    assert rel_err(ref, O.matmul(A, np.ascontiguousarray(B.T).reshape(7, 6))) > 1e-2


def test_gemm_attributes():
    rng = np.random.default_rng(2)
    A = rng.normal(size=(6, 4)).astype(np.float32)
    B = rng.normal(size=(6, 5)).astype(np.float32)
    C = rng.normal(size=(4, 5)).astype(np.float32)
    ref = 0.5 * (A.astype(np.float64).T @ B.astype(np.float64)) + 2.0 * C
    assert rel_err(ref, O.gemm(A, B, C, alpha=0.5, beta=2.0, transA=1, transB=0)) < TOL


# ----------------------------------------------------------------------------- conv
@pytest.mark.parametrize("num_in_channels, kernel_size, num_filters, bias",
                         [(1, (3, 3), 8, True), (8, (3, 3), 3, False), (8, (5, 5), 3, True), (8, (4, 4), 3, False)])
def test_conv_reference_test_grid(num_in_channels, kernel_size, num_filters, bias):
    # the parameter grid of the reference's test_conv_simple (test_conv_expansion.py:10-13)
    rng = np.random.default_rng(3)
    X = rng.random((8, num_in_channels, 32, 32)).astype(np.float32)
    W = rng.random((num_filters, num_in_channels, *kernel_size)).astype(np.float32)
    B = rng.random(num_filters).astype(np.float32) if bias else None
    ref = F.conv2d(torch.from_numpy(X).double(), torch.from_numpy(W).double(),
                   bias=None if B is None else torch.from_numpy(B).double()).numpy()
    assert rel_err(ref, O.conv2d(X, W, B)) < TOL


@pytest.mark.parametrize("strides, pads, dil", [((2, 2), (0, 0, 0, 0), (1, 1)), ((1, 1), (1, 1, 1, 1), (1, 1)),
                                                ((2, 3), (2, 0, 1, 3), (1, 1)), ((1, 2), (1, 2, 2, 1), (2, 3))])
def test_conv_stride_pad_dilation_vs_torch_and_bruteforce(strides, pads, dil):
    rng = np.random.default_rng(4)
    X = rng.normal(size=(2, 3, 11, 13)).astype(np.float32)
    W = rng.normal(size=(4, 3, 3, 2)).astype(np.float32)
    B = rng.normal(size=4).astype(np.float32)
    xp = F.pad(torch.from_numpy(X).double(), (pads[1], pads[3], pads[0], pads[2]))
    ref = F.conv2d(xp, torch.from_numpy(W).double(), torch.from_numpy(B).double(), stride=strides,
                   dilation=dil).numpy()
    y = O.conv2d(X, W, B, strides, pads, dil)
    assert y.shape == ref.shape == O.conv_output_shape(X.shape, W.shape, strides, pads, dil)
    assert rel_err(ref, y) < TOL
    assert rel_err(ref, O.conv2d_bruteforce(X, W, B, strides, pads, dil)) < 1e-12 + TOL


def test_conv_stride_is_not_ignored():
    # PureConv2D drops the stride (img_op_implementations.py:278); the parity target keeps it
    rng = np.random.default_rng(5)
    X = rng.random((1, 1, 8, 8)).astype(np.float32)
    W = rng.random((1, 1, 3, 3)).astype(np.float32)
    full = O.conv2d(X, W)
    strided = O.conv2d(X, W, strides=(2, 2))
    assert strided.shape == (1, 1, 3, 3)
    assert np.allclose(strided, full[:, :, ::2, ::2])


# ----------------------------------------------------------------------------- softmax / layernorm / gelu
@pytest.mark.parametrize("axis", [0, 1, -1])
def test_softmax_vs_torch(axis):
    rng = np.random.default_rng(6)
    X = rng.normal(scale=10, size=(2, 4, 10)).astype(np.float32)  # the reference's case (test_expansions.py:347)
    ref = F.softmax(torch.from_numpy(X).double(), dim=axis).numpy()
    y = O.softmax(X, axis=axis)
    assert np.linalg.norm(ref - y) < 1e-5  # the reference's own bar (test_expansions.py:379)
    assert rel_err(ref, y) < TOL


def test_softmax_invariants():
    rng = np.random.default_rng(7)
    X = rng.normal(size=(6, 128)).astype(np.float32)
    y = O.softmax(X)
    assert np.allclose(y.sum(-1), 1.0, atol=1e-6)
    assert np.allclose(O.softmax(X + 3.0), y, atol=1e-6)          # shift invariance
    assert np.allclose(O.softmax(np.full((2, 5), 4.0, np.float32)), 0.2)  # constant row -> 1/n
    big = np.array([[1000.0, 0.0]], np.float32)                    # max subtraction keeps it finite
    assert np.allclose(O.softmax(big), [[1.0, 0.0]])


def test_layernorm_vs_torch_and_special_cases():
    rng = np.random.default_rng(8)
    X = rng.normal(size=(4, 9, 48)).astype(np.float32)
    g = rng.normal(1, 0.1, size=48).astype(np.float32)
    b = rng.normal(0, 0.1, size=48).astype(np.float32)
    ref = F.layer_norm(torch.from_numpy(X).double(), (48, ), torch.from_numpy(g).double(),
                       torch.from_numpy(b).double(), eps=1e-12).numpy()
    assert rel_err(ref, O.layer_normalization(X, g, b, epsilon=1e-12)) < TOL
    # two trailing axes
    g2 = rng.normal(1, 0.1, size=(9, 48)).astype(np.float32)
    ref2 = F.layer_norm(torch.from_numpy(X).double(), (9, 48), torch.from_numpy(g2).double(), None, eps=1e-5).numpy()
    assert rel_err(ref2, O.layer_normalization(X, g2, None, axis=1, epsilon=1e-5)) < TOL
    # gamma = 1, beta = 0 -> zero mean, unit (biased) variance
    y = O.layer_normalization(X, np.ones(48, np.float32), np.zeros(48, np.float32), epsilon=1e-12)
    assert np.allclose(y.mean(-1), 0, atol=1e-6) and np.allclose(y.var(-1), 1, atol=1e-4)
    # constant row -> beta
    c = O.layer_normalization(np.full((1, 48), 7.0, np.float32), g, b, epsilon=1e-5)
    assert np.allclose(c, b, atol=1e-6)


def test_gelu_erf_relu_closed_forms():
    x = np.linspace(-6, 6, 101).astype(np.float32)
    ref = np.array([0.5 * v * (1 + math.erf(v / math.sqrt(2))) for v in x.astype(np.float64)])
    assert rel_err(ref, O.gelu(x)) < TOL
    assert rel_err(F.gelu(torch.from_numpy(x).double()).numpy(), O.gelu(x)) < TOL
    assert rel_err(np.array([math.erf(v) for v in x.astype(np.float64)]), O.erf(x)) < TOL
    assert np.array_equal(O.relu(x), np.where(x > 0, x, 0).astype(np.float32))
    assert O.relu(x).dtype == np.float32


def test_unary_maps_closed_forms():
    """Log, Tanh, Reciprocal, Softplus, Sigmoid (and Exp, Neg, Abs) against the math module in double, value
    by value, plus what fixes the formula: the reference's Softplus is log(1 + exp(x)) literally, so it
    overflows at x = 89 and is exactly 0 where exp(x) is below half an ulp of 1."""
    rng = np.random.default_rng(21)
    x = rng.normal(scale=3, size=500).astype(np.float32)
    x64 = x.astype(np.float64)
    each = lambda f, v: np.array([f(t) for t in v])
    assert np.allclose(O.tanh(x), each(math.tanh, x64), rtol=3e-7, atol=1e-7)
    assert np.allclose(O.log(np.abs(x) + 0.1), each(math.log, np.abs(x).astype(np.float32).astype(np.float64) + np.float32(0.1)),
                       rtol=1e-6, atol=2e-7)
    assert np.allclose(O.reciprocal(x), 1.0 / x64, rtol=2e-7)
    assert np.allclose(O.softplus(x), each(lambda t: math.log1p(math.exp(t)), x64), rtol=1e-6, atol=1e-7)
    assert np.allclose(O.sigmoid(x), each(lambda t: 1.0 / (1.0 + math.exp(-t)), x64), rtol=3e-7)
    assert np.allclose(O.sigmoid(x) + O.sigmoid(-x), 1.0, atol=2e-7)        # symmetry
    assert np.allclose(O.exp(x), each(math.exp, x64), rtol=3e-7)
    assert np.array_equal(O.neg(x), -x) and np.array_equal(O.abs(x), np.abs(x))
    assert O.tanh(x).dtype == O.softplus(x).dtype == O.sigmoid(x).dtype == O.reciprocal(x).dtype == np.float32
    edge = np.array([89.0, -20.0, 0.0], dtype=np.float32)
    sp = O.softplus(edge)
    assert np.isinf(sp[0]) and sp[1] == 0.0 and sp[2] == np.float32(math.log(2.0))
    assert O.sigmoid(np.array([-100.0, 100.0], np.float32)).tolist() == [0.0, 1.0]


def test_reductions_log_softmax_sum_closed_forms():
    """ReduceSum / Max / Min against explicit loops, LogSoftmax against log(softmax) in double and its
    normalisation, Sum against left-to-right addition."""
    rng = np.random.default_rng(22)
    x = rng.normal(size=(3, 5, 7)).astype(np.float32)
    s = O.reduce_sum(x, [1], keepdims=0)
    assert s.shape == (3, 7) and s.dtype == np.float32
    for i in range(3):
        for k in range(7):
            col = [float(x[i, j, k]) for j in range(5)]
            assert abs(s[i, k] - math.fsum(col)) < 1e-5
            assert O.reduce_max(x, [1], 0)[i, k] == max(col) and O.reduce_min(x, [1], 0)[i, k] == min(col)
    assert O.reduce_max(x, [0, 2]).shape == (1, 5, 1) and O.reduce_sum(x, [0, 1, 2], keepdims=0).shape == ()
    ls = O.log_softmax(x, axis=1)
    assert np.allclose(ls, np.log(O.softmax(x.astype(np.float64), axis=1)), atol=1e-6)
    assert np.allclose(np.exp(ls.astype(np.float64)).sum(1), 1.0, atol=1e-6)
    assert np.allclose(O.log_softmax(x + 100.0, axis=1), ls, atol=1e-4)        # shift invariance
    assert np.allclose(O.log_softmax(np.zeros((2, 8), np.float32)), -math.log(8.0))
    a, b, c = (rng.normal(size=(4, 4)).astype(np.float32) for _ in range(3))
    assert np.array_equal(O.sum_(a, b, c), (a + b) + c) and np.array_equal(O.sum_(a), a)


@pytest.mark.parametrize("kernel, strides, pads, dil", [((2, 2), (2, 2), (0, 0, 0, 0), (1, 1)), ((3, 3), (2, 2), (1, 1, 1, 1), (1, 1)),
                                                        ((3, 2), (1, 2), (1, 0, 2, 1), (1, 1)), ((2, 3), (1, 1), (0, 1, 0, 1), (2, 2))])
def test_maxpool_global_average_pool_batchnorm_vs_torch(kernel, strides, pads, dil):
    """MaxPool against torch's max_pool2d (symmetric pads) and a brute-force window loop (any pads);
    GlobalAveragePool and inference BatchNormalization against torch and their closed forms."""
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(26)
    x = rng.normal(size=(2, 3, 9, 11)).astype(np.float32)
    got = O.maxpool2d(x, kernel, strides, pads, dil)
    if pads[0] == pads[2] and pads[1] == pads[3]:
        ref = F.max_pool2d(torch.from_numpy(x), kernel, strides, (pads[0], pads[1]), dil).numpy()
        assert np.array_equal(got, ref)
    eh, ew = (kernel[0] - 1) * dil[0] + 1, (kernel[1] - 1) * dil[1] + 1
    for oh in range(got.shape[2]):
        for ow in range(got.shape[3]):
            best = np.full((2, 3), -np.inf, np.float32)
            for kh in range(kernel[0]):
                for kw in range(kernel[1]):
                    ih, iw = oh * strides[0] - pads[0] + kh * dil[0], ow * strides[1] - pads[1] + kw * dil[1]
                    if 0 <= ih < 9 and 0 <= iw < 11:
                        best = np.maximum(best, x[:, :, ih, iw])
            assert np.array_equal(got[:, :, oh, ow], best)
    assert got.shape[2:] == ((9 + pads[0] + pads[2] - eh) // strides[0] + 1, (11 + pads[1] + pads[3] - ew) // strides[1] + 1)
    gap = O.global_average_pool(x)
    assert gap.shape == (2, 3, 1, 1) and np.allclose(gap, F.adaptive_avg_pool2d(torch.from_numpy(x), 1).numpy(), atol=1e-6)
    scale, b, mean = (rng.normal(size=3).astype(np.float32) for _ in range(3))
    var = rng.uniform(0.5, 2.0, size=3).astype(np.float32)
    bn = O.batch_normalization(x, scale, b, mean, var, 1e-5)
    ref = F.batch_norm(torch.from_numpy(x), torch.from_numpy(mean), torch.from_numpy(var), torch.from_numpy(scale),
                       torch.from_numpy(b), training=False, eps=1e-5).numpy()
    assert np.allclose(bn, ref, rtol=1e-5, atol=1e-6)
    # identity statistics leave x unchanged up to eps; zero scale gives the bias
    ident = O.batch_normalization(x, np.ones(3, np.float32), np.zeros(3, np.float32), np.zeros(3, np.float32), np.ones(3, np.float32), 0.0)
    assert np.array_equal(ident, x)
    assert np.array_equal(O.batch_normalization(x, np.zeros(3, np.float32), b, mean, var)[0, :, 0, 0], b)


def test_pow_and_reduce_mean_closed_forms():
    rng = np.random.default_rng(21)
    x = rng.normal(size=(3, 5, 7)).astype(np.float32)
    assert np.array_equal(O.pow(x, 2.0), x * x)                                    # the exponent of the exported LayerNorm
    pos = np.abs(x) + 0.5
    ref = np.array([math.pow(float(v), 1.5) for v in pos.reshape(-1)]).reshape(pos.shape)
    assert rel_err(ref, O.pow(pos, np.float32(1.5))) < TOL
    m = O.reduce_mean(x, [-1])
    assert m.shape == (3, 5, 1) and m.dtype == np.float32
    brute = np.array([[sum(float(v) for v in x[i, j]) / 7 for j in range(5)] for i in range(3)])
    assert rel_err(brute, m[..., 0]) < TOL
    assert O.reduce_mean(x, [1, 2], keepdims=0).shape == (3, ) and O.reduce_mean(x, [0], keepdims=1).shape == (1, 5, 7)
    assert np.allclose(O.reduce_mean(np.full((4, 6), 2.5, np.float32), [1]), 2.5)


def test_add_broadcasting():
    rng = np.random.default_rng(9)
    a = rng.normal(size=(8, 16, 24)).astype(np.float32)
    b = rng.normal(size=(24, )).astype(np.float32)
    assert np.array_equal(O.add(a, b), a + b[None, None, :])
    assert O.add(a, a).shape == a.shape


# ----------------------------------------------------------------------------- matmul integer
def test_matmul_integer_identity_and_extremes():
    rng = np.random.default_rng(10)
    A = rng.integers(-128, 128, size=(33, 70), dtype=np.int8)
    B = rng.integers(-128, 128, size=(70, 21), dtype=np.int8)
    za, zb = 3, -2
    y = O.matmul_integer(A, B, za, zb)
    a64, b64 = A.astype(np.int64), B.astype(np.int64)
    ident = a64 @ b64 - zb * a64.sum(1, keepdims=True) - za * b64.sum(0, keepdims=True) + 70 * za * zb
    assert np.array_equal(y, ident.astype(np.int32))
    # brute force on one row
    row = [sum((int(A[0, k]) - za) * (int(B[k, j]) - zb) for k in range(70)) for j in range(21)]
    assert np.array_equal(y[0], np.array(row, dtype=np.int32))
    # extreme values: (-128 - 127) * (-128 - 127) * K
    Ae = np.full((2, 768), -128, np.int8)
    Be = np.full((768, 2), -128, np.int8)
    assert np.all(O.matmul_integer(Ae, Be, 127, 127) == 768 * 255 * 255)
    # swapping the zero points must change the result
    assert not np.array_equal(y, O.matmul_integer(A, B, zb, za))


def test_matmul_integer_unsigned_operands_and_zero_point_vectors(c_oracle):
    """uint8 operands and one zero point per row of A / per column of B (ONNX MatMulInteger, T1 and T2 in
    {int8, uint8}): brute force in Python integers, the row/column-sum identity, and the case that must
    reduce to the signed one (u - 128 as int8 with the zero point moved by 128)."""
    rng = np.random.default_rng(21)
    M, K, N = 9, 37, 11
    for a_dt, b_dt in ((np.uint8, np.int8), (np.int8, np.uint8), (np.uint8, np.uint8)):
        lo_a, hi_a = (0, 256) if a_dt == np.uint8 else (-128, 128)
        lo_b, hi_b = (0, 256) if b_dt == np.uint8 else (-128, 128)
        A = rng.integers(lo_a, hi_a, size=(M, K)).astype(a_dt)
        B = rng.integers(lo_b, hi_b, size=(K, N)).astype(b_dt)
        za = rng.integers(lo_a, hi_a, size=M).astype(a_dt)
        zb = rng.integers(lo_b, hi_b, size=N).astype(b_dt)
        y = O.matmul_integer(A, B, za, zb)
        brute = [[sum((int(A[m, k]) - int(za[m])) * (int(B[k, n]) - int(zb[n])) for k in range(K)) for n in range(N)]
                 for m in range(M)]
        assert np.array_equal(y, np.array(brute, dtype=np.int64).astype(np.int32))
        assert np.array_equal(y, c_oracle.matmul_integer(A, B, za, zb))
        a64, b64, za64, zb64 = A.astype(np.int64), B.astype(np.int64), za.astype(np.int64)[:, None], zb.astype(np.int64)[None, :]
        ident = a64 @ b64 - zb64 * a64.sum(1, keepdims=True) - za64 * b64.sum(0, keepdims=True) + K * za64 * zb64
        assert np.array_equal(y, ident.astype(np.int32))
        # scalar zero points of the operand's type
        ys = O.matmul_integer(A, B, za[0], zb[0])
        assert np.array_equal(ys, c_oracle.matmul_integer(A, B, za[0], zb[0]))
        assert np.array_equal(ys[0], y[0] if N == 1 else np.array([sum((int(A[0, k]) - int(za[0])) * (int(B[k, n]) - int(zb[0]))
                                                                      for k in range(K)) for n in range(N)], dtype=np.int32))
    # reduction to the signed case
    Au = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    Bs = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
    As = (Au.astype(np.int16) - 128).astype(np.int8)
    assert np.array_equal(O.matmul_integer(Au, Bs, np.uint8(200), np.int8(-5)), O.matmul_integer(As, Bs, np.int8(72), np.int8(-5)))
    # extreme values: (255 - 0) * (255 - 0) * K and (0 - 255)(255 - 0) K stay inside int32 for K = 768
    Ae, Be = np.full((2, 768), 255, np.uint8), np.full((768, 2), 255, np.uint8)
    assert np.all(O.matmul_integer(Ae, Be) == 768 * 255 * 255)
    assert np.all(O.matmul_integer(np.zeros_like(Ae), Be, np.uint8(255), np.uint8(0)) == -768 * 255 * 255)
    # a stack of matrices with a per-row zero point of shape [D, M, 1]
    A3 = rng.integers(0, 256, size=(2, M, K)).astype(np.uint8)
    z3 = rng.integers(0, 256, size=(2, M, 1)).astype(np.uint8)
    y3 = O.matmul_integer(A3, Bs, z3, np.int8(4))
    for d in range(2):
        assert np.array_equal(y3[d], O.matmul_integer(A3[d], Bs, z3[d, :, 0], np.int8(4)))


# ----------------------------------------------------------------------------- C restatement vs numpy restatement
def test_c_oracle_matches_numpy_oracle(c_oracle):
    rng = np.random.default_rng(11)
    X = rng.normal(size=(3, 5, 12, 10)).astype(np.float32)
    W = rng.normal(size=(6, 5, 3, 3)).astype(np.float32)
    B = rng.normal(size=6).astype(np.float32)
    for strides, pads, dil in (((1, 1), (1, 1, 1, 1), (1, 1)), ((2, 2), (0, 0, 0, 0), (1, 1)), ((2, 1), (1, 0, 2, 1), (1, 2))):
        assert rel_err(O.conv2d(X, W, B, strides, pads, dil), c_oracle.conv2d(X, W, B, strides, pads, dil)) < 1e-5
    x = rng.normal(size=(7, 128)).astype(np.float32)
    assert rel_err(O.softmax(x), c_oracle.softmax(x)) < 1e-6
    g = rng.normal(1, 0.02, size=128).astype(np.float32)
    b = rng.normal(0, 0.02, size=128).astype(np.float32)
    assert rel_err(O.layer_normalization(x, g, b, epsilon=1e-12), c_oracle.layer_normalization(x, g, b, 1e-12)) < 1e-5
    assert rel_err(O.gelu(x), c_oracle.gelu(x)) < 1e-6
    A = rng.integers(-128, 128, size=(17, 40), dtype=np.int8)
    Bm = rng.integers(-128, 128, size=(40, 23), dtype=np.int8)
    assert np.array_equal(O.matmul_integer(A, Bm, 3, -2), c_oracle.matmul_integer(A, Bm, 3, -2))
    a = rng.normal(size=(9, 14)).astype(np.float32)
    bb = rng.normal(size=(14, 11)).astype(np.float32)
    assert rel_err(O.matmul(a, bb), c_oracle.matmul(a, bb)) < 1e-5


def test_bert_layer_against_transformers():
    """The composition is the module the reference tests (BertLayer, test_bert_encoder.py:17)."""
    from transformers import BertConfig
    from transformers.models.bert.modeling_bert import BertLayer
    hidden, heads, ffn, bsz, seq = 64, 4, 128, 2, 12
    cfg = BertConfig(hidden_size=hidden, num_attention_heads=heads, intermediate_size=ffn, hidden_act="gelu",
                     layer_norm_eps=1e-12, attention_probs_dropout_prob=0.0, hidden_dropout_prob=0.0)
    cfg._attn_implementation = "eager"
    layer = BertLayer(cfg).eval()
    rng = np.random.default_rng(12)
    w = O.bert_layer_weights(rng, hidden=hidden, ffn=ffn)
    for k in ("bq", "bk", "bv", "bo", "b1", "b2"):
        w[k] = rng.normal(0, 0.02, size=w[k].shape).astype(np.float32)
    x = rng.normal(size=(bsz, seq, hidden)).astype(np.float32)
    t = torch.from_numpy
    with torch.no_grad():
        att, so = layer.attention.self, layer.attention.output
        for lin, wn, bn in ((att.query, "wq", "bq"), (att.key, "wk", "bk"), (att.value, "wv", "bv"),
                            (so.dense, "wo", "bo"), (layer.intermediate.dense, "w1", "b1"),
                            (layer.output.dense, "w2", "b2")):
            lin.weight.copy_(t(w[wn]).T)
            lin.bias.copy_(t(w[bn]))
        so.LayerNorm.weight.copy_(t(w["ln1_g"])); so.LayerNorm.bias.copy_(t(w["ln1_b"]))
        layer.output.LayerNorm.weight.copy_(t(w["ln2_g"])); layer.output.LayerNorm.bias.copy_(t(w["ln2_b"]))
        ref = layer(t(x))
        ref = (ref[0] if isinstance(ref, (tuple, list)) else ref).numpy()
    assert rel_err(ref, O.bert_layer(x, w, heads=heads)) < 5e-6


# ----------------------------------------------------------------------------- Slice, Cast, Einsum (checker functions of the widening operators)
def _onnx_slice_indices(dim, start, end, step):
    """Index list of one axis by the ONNX Slice rules, written out without Python slicing: negative start / end
    count from the end, then start is clamped to [0, dim] (step > 0) or [0, dim - 1] (step < 0) and end to
    [0, dim] or [-1, dim - 1]."""
    assert step != 0
    if start < 0:
        start += dim
    if end < 0:
        end += dim
    if step > 0:
        start = min(max(start, 0), dim)
        end = min(max(end, 0), dim)
    else:
        start = min(max(start, 0), dim - 1)
        end = min(max(end, -1), dim - 1)
    out, i = [], start
    while (i < end) if step > 0 else (i > end):
        out.append(i)
        i += step
    return out


def test_slice_against_explicit_index_loops():
    INT64_MAX, INT64_MIN = 2**63 - 1, -2**63
    rng = np.random.default_rng(40)
    data = rng.normal(size=(5, 7, 4)).astype(np.float32)
    cases = [
        ([1], [4], None, None), ([0], [INT64_MAX], [0], None), ([2], [INT64_MAX], [1], [1]),
        ([-3], [INT64_MAX], [1], [1]), ([1, 0], [100, -1], [0, 2], [1, 1]), ([0, 1, 1], [5, 7, 3], [0, 1, 2], [2, 3, 1]),
        ([6], [0], [1], [-1]), ([6], [INT64_MIN], [1], [-1]), ([-1], [INT64_MIN], [1], [-2]), ([100], [-100], [1], [-3]),
        ([3], [3], [0], [1]), ([4], [2], [0], [1]), ([-100], [2], [0], [1]), ([1], [3], [-1], [1]), ([3, 5], [0, 1], [-1, -2], [-1, -2]),
    ]
    for starts, ends, axes, steps in cases:
        ax = list(range(len(starts))) if axes is None else [a % data.ndim for a in axes]
        st = [1] * len(starts) if steps is None else steps
        picks = [list(range(d)) for d in data.shape]
        for s, e, a, t in zip(starts, ends, ax, st):
            picks[a] = _onnx_slice_indices(data.shape[a], s, e, t)
        expected = np.empty([len(p) for p in picks], np.float32)
        for i, pi in enumerate(picks[0]):
            for j, pj in enumerate(picks[1]):
                for k, pk in enumerate(picks[2]):
                    expected[i, j, k] = data[pi, pj, pk]
        got = O.slice_(data, starts, ends, axes, steps)
        assert got.shape == expected.shape and np.array_equal(got, expected), (starts, ends, axes, steps)


def test_cast_truncates_toward_zero_and_to_bool():
    x = np.array([0.5, -0.5, 1.5, -1.5, 2.9, -2.9, 3.0, -3.0, 0.0, -0.0, 1e-30, 255.9, -128.9, 65536.7], np.float32)
    toward_zero = [int(v) for v in x.tolist()]   # Python's int() truncates toward zero
    assert toward_zero[:8] == [0, 0, 1, -1, 2, -2, 3, -3]
    assert O.cast(x, np.int32).tolist() == toward_zero
    assert O.cast(x, np.int64).tolist() == toward_zero
    assert O.cast(x[:12], np.int16).tolist() == toward_zero[:12]
    assert O.cast(x, np.bool_).tolist() == [v != 0 for v in x.tolist()]
    i = np.array([-2**24, -1, 0, 1, 2**24, 123456], np.int32)
    assert O.cast(i, np.float32).tolist() == [float(v) for v in i.tolist()] and O.cast(i, np.float32).dtype == np.float32
    assert O.cast(np.array([True, False]), np.float32).tolist() == [1.0, 0.0]
    d = np.array([1.0 + 2.0**-30, 0.1], np.float64)
    assert O.cast(d, np.float32).tolist() == [1.0, float(np.float32(0.1))]


def _einsum_brute(equation, a, b):
    ins, out = equation.replace(" ", "").split("->")
    ia, ib = ins.split(",")
    size = {}
    for letters, arr in ((ia, a), (ib, b)):
        for letter, n in zip(letters, arr.shape):
            assert size.setdefault(letter, n) == n
    letters = sorted(size)
    result = np.zeros([size[c] for c in out], np.float64)
    idx = dict.fromkeys(letters, 0)

    def walk(depth):
        if depth == len(letters):
            result[tuple(idx[c] for c in out)] += float(a[tuple(idx[c] for c in ia)]) * float(b[tuple(idx[c] for c in ib)])
            return
        for v in range(size[letters[depth]]):
            idx[letters[depth]] = v
            walk(depth + 1)

    walk(0)
    return result


def test_einsum_against_brute_force_index_loops():
    rng = np.random.default_rng(41)
    shapes = {"i": 3, "j": 4, "k": 2, "b": 2, "h": 3, "d": 4}
    for eq in ("ik,kj->ij", "bik,kj->bij", "bik,bkj->bij", "bhid,bhjd->bhij", "ik,jk->ij", "ki,kj->ji", "bij,bjk->bki",
               "i,i->i", "ij,j->i"):
        ia, ib = eq.split("->")[0].split(",")
        a = rng.normal(size=[shapes[c] for c in ia]).astype(np.float32)
        b = rng.normal(size=[shapes[c] for c in ib]).astype(np.float32)
        got = O.einsum(eq, a, b)
        want = _einsum_brute(eq, a, b)
        assert got.shape == want.shape and np.allclose(got, want, rtol=1e-5, atol=1e-6), eq
    # a transposed operand or a swapped output must not go unnoticed
    a, b = rng.normal(size=(3, 3)).astype(np.float32), rng.normal(size=(3, 3)).astype(np.float32)
    assert not np.allclose(O.einsum("ik,kj->ij", a, b), _einsum_brute("ik,jk->ij", a, b))
    assert not np.allclose(O.einsum("ik,kj->ij", a, b), _einsum_brute("ik,kj->ji", a, b))


def test_elementwise_pass_throughs_against_the_math_module():
    """sub, mul, div, sqrt are one-line numpy calls in the checker; pin them value by value."""
    import math
    rng = np.random.default_rng(42)
    a = rng.normal(size=(3, 5)).astype(np.float32)
    b = (rng.normal(size=5) + 3).astype(np.float32)
    for name, fn in (("sub", lambda x, y: x - y), ("mul", lambda x, y: x * y), ("div", lambda x, y: x / y)):
        got = getattr(O, name)(a, b)
        for i in range(3):
            for j in range(5):
                assert got[i, j] == np.float32(fn(np.float32(a[i, j]), np.float32(b[j]))), name
    s = O.sqrt(np.abs(a))
    for i in range(3):
        for j in range(5):
            assert abs(float(s[i, j]) - math.sqrt(abs(float(a[i, j])))) <= 1e-7 * max(1.0, float(s[i, j]))

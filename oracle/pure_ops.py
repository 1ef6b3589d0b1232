"""CPU restatement of the reference's ONNX expansions -- TEST INFRASTRUCTURE ONLY.

This package is the checker for the HIP kernels: it may be imported by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``, never by the product package. Each function restates, in numpy,
what the reference's CPU ("pure") expansion computes for one ONNX node, pass by
pass, and cites the lines it follows. Where the reference has no expansion of
its own (MatMulInteger runs inside ONNX Runtime, LayerNormalization and Gelu
exist only as exporter decompositions) the ONNX operator specification is
restated instead and the docstring says so.

How each function is pinned (tests/test_oracle.py):
  matmul / gemm        numpy ``@`` in float64, brute-force triple loop on small shapes
                       (the reference's own check is ``np.allclose(X @ Z, result)``,
                       tests/pure_expansions/test_expansions.py:29,56)
  conv2d               torch.nn.functional.conv2d, the reference's comparator
                       (tests/pure_expansions/test_conv_expansion.py:30-35), with
                       stride / pad / dilation; brute-force seven-loop on small shapes
  softmax              torch.nn.functional.softmax (test_expansions.py:349); rows sum
                       to 1, shift invariance, constant row -> 1/n
  layer_normalization  torch.nn.functional.layer_norm; constant row -> beta;
                       gamma=1, beta=0 -> zero mean, unit variance
  gelu                 math.erf closed form, torch gelu
  relu / add / ...     closed forms, numpy broadcasting
  matmul_integer       int64 closed form and the rowsum/colsum identity;
                       "parity unpinned" against the reference itself: the reference
                       delegates this op to a patched ONNX Runtime binary that is not
                       part of its source tree, and none of its tests touch the op
  bert_layer           transformers.BertLayer (the module the reference tests,
                       tests/pytorch/test_bert_encoder.py:17) with the same weights
plus the committed fixtures under tests/golden/.
"""
import itertools
import math

import numpy as np

# --------------------------------------------------------------------------- contractions


def matmul_einsum_string(a_ndim: int, b_ndim: int) -> str:
    """The einsum PureMatMul builds (pure_implementations.py:151-210): 'ik,kj->ij'
    plus one letter per leading dimension, taken from z, y, x, ... and aligned
    from the right so that missing leading dims broadcast."""
    if a_ndim < 2 or b_ndim < 2:
        raise ValueError("1-D operands are refused by PureMatMul (pure_implementations.py:133-140)")
    letters = [chr(ord('z') - i) for i in range(26)]
    letters = [l for l in letters if l not in ['i', 'j', 'k']]
    arg1, arg2, result = 'ik', 'kj', 'ij'
    for dim0, dim1 in itertools.zip_longest(reversed(range(a_ndim - 2)), reversed(range(b_ndim - 2))):
        letter = letters.pop()
        if dim0 is not None:
            arg1 = letter + arg1
        if dim1 is not None:
            arg2 = letter + arg2
        result = letter + result
    return '{},{}->{}'.format(arg1, arg2, result)


def matmul(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    """ONNXMatMul as PureMatMul -> ONNXEinsum -> create_einsum_sdfg
    (pure_implementations.py:130-267). Size-1 leading dims broadcast like numpy."""
    eq = matmul_einsum_string(A.ndim, B.ndim)
    batch = np.broadcast_shapes(A.shape[:-2], B.shape[:-2])
    A = np.broadcast_to(A, batch[len(batch) - (A.ndim - 2):] + A.shape[-2:])
    B = np.broadcast_to(B, batch[len(batch) - (B.ndim - 2):] + B.shape[-2:])
    return np.einsum(eq, A, B, optimize=True).astype(A.dtype, copy=False)


def gemm(A, B, C=None, alpha=1.0, beta=1.0, transA=0, transB=0):
    """ONNX Gemm. PureGemm (pure_implementations.py:433-459) computes
    ``A @ B.T + C`` and accepts only alpha=1, beta=1, transA=0, transB=1; the other
    attribute values follow the operator specification."""
    a = A.T if transA else A
    b = B.T if transB else B
    y = (a @ b) * np.asarray(alpha, dtype=A.dtype)
    if C is not None:
        y = y + np.asarray(beta, dtype=A.dtype) * C
    return y.astype(A.dtype, copy=False)


def matmul_integer(A, B, a_zero_point=0, b_zero_point=0):
    """ONNX MatMulInteger (opset 10): ``(A - a_zp) @ (B - b_zp)`` accumulated in
    int32, operands int8 or uint8. ``a_zero_point`` is one value or one per row of
    A (``[M]`` for a matrix, ``[..., M, 1]`` for a stack), ``b_zero_point`` one
    value or one per column of B (``[N]``). The reference expands this node only
    through ONNX Runtime (onnx_op.py:686-687); this is the specification's formula,
    evaluated in int64 and wrapped to int32."""
    a_zp = np.asarray(a_zero_point).astype(np.int64)
    if a_zp.ndim == 1 and a_zp.size > 1:
        a_zp = a_zp.reshape(-1, 1)
    b_zp = np.asarray(b_zero_point).astype(np.int64)
    a = A.astype(np.int64) - a_zp
    b = B.astype(np.int64) - b_zp
    return (a @ b).astype(np.int32)


# --------------------------------------------------------------------------- convolution


def conv_output_shape(x_shape, w_shape, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1)):
    n, _, h, w = x_shape
    m, _, kh, kw = w_shape
    oh = (h + pads[0] + pads[2] - ((kh - 1) * dilations[0] + 1)) // strides[0] + 1
    ow = (w + pads[1] + pads[3] - ((kw - 1) * dilations[1] + 1)) // strides[1] + 1
    return n, m, oh, ow


def conv2d(X, W, B=None, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1)):
    """ONNXConv, 2-D, group 1. Same pass structure as PureConv2D
    (img_op_implementations.py:246-293): the output is initialised with zero
    (``zero_init``) or the broadcast bias (``broadcast``), then every
    (cin, hx, hy) term is accumulated into it; the loops over (cin, hx, hy) are
    explicit, the four outer map dimensions are numpy slices.

    The reference indexes ``X[b, cin, hx + out_x, hy + out_y]`` (:278, :291), i.e.
    it drops the stride and refuses any pad (:201-203). The stride, pad and
    dilation terms of the ONNX specification are restored here, which is what the
    reference computes through its default ONNX Runtime implementation and what its
    stride-2 example expects (examples/plot_conv.py:43-46)."""
    n, c, h, w = X.shape
    m, c2, kh, kw = W.shape
    assert c == c2
    _, _, oh, ow = conv_output_shape(X.shape, W.shape, strides, pads, dilations)
    xp = np.zeros((n, c, h + pads[0] + pads[2], w + pads[1] + pads[3]), dtype=X.dtype)
    xp[:, :, pads[0]:pads[0] + h, pads[1]:pads[1] + w] = X
    Y = np.zeros((n, m, oh, ow), dtype=X.dtype)
    if B is not None:
        Y += B.reshape(1, m, 1, 1)
    for cin in range(c):
        for hx in range(kh):
            for hy in range(kw):
                y0, x0 = hx * dilations[0], hy * dilations[1]
                patch = xp[:, cin, y0:y0 + (oh - 1) * strides[0] + 1:strides[0],
                           x0:x0 + (ow - 1) * strides[1] + 1:strides[1]]
                Y += W[:, cin, hx, hy].reshape(1, m, 1, 1) * patch[:, None, :, :]
    return Y


def conv2d_bruteforce(X, W, B=None, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1)):
    """The seven nested loops of img_op_implementations.py:270-293 written out in
    plain Python (small shapes only), with the ONNX stride/pad/dilation terms."""
    n, c, h, w = X.shape
    m, _, kh, kw = W.shape
    _, _, oh, ow = conv_output_shape(X.shape, W.shape, strides, pads, dilations)
    Y = np.zeros((n, m, oh, ow), dtype=np.float64)
    for b in range(n):
        for f in range(m):
            for oy in range(oh):
                for ox in range(ow):
                    acc = 0.0 if B is None else float(B[f])
                    for cin in range(c):
                        for hx in range(kh):
                            for hy in range(kw):
                                iy = oy * strides[0] - pads[0] + hx * dilations[0]
                                ix = ox * strides[1] - pads[1] + hy * dilations[1]
                                if 0 <= iy < h and 0 <= ix < w:
                                    acc += float(W[f, cin, hx, hy]) * float(X[b, cin, iy, ix])
                    Y[b, f, oy, ox] = acc
    return Y


# --------------------------------------------------------------------------- reductions


def softmax(X, axis=-1):
    """PureSoftmax, the five statements of pure_implementations.py:358-364."""
    reduced_shape = list(X.shape)
    reduced_shape[axis] = 1
    max_ = np.max(X, axis=axis)
    max_keepdims = np.reshape(max_, reduced_shape)
    exp_arr = np.exp(X - max_keepdims)
    sum_ = np.sum(exp_arr, axis=axis)
    sum_keepdims = np.reshape(sum_, reduced_shape)
    return exp_arr / sum_keepdims


def reduce_mean(data, axes, keepdims=1):
    """PureReduceMean (pure_implementations.py:97-109)."""
    return np.mean(data, axis=tuple(axes), keepdims=bool(keepdims)).astype(data.dtype, copy=False)


def reduce_sum(data, axes, keepdims=1):
    """PureReduceSum: np.sum over ``axes`` (pure_implementations.py:301-313)."""
    return np.sum(data, axis=tuple(axes), keepdims=bool(keepdims)).astype(data.dtype, copy=False)


def reduce_max(data, axes, keepdims=1):
    """PureReduceMax: np.max over ``axes`` (pure_implementations.py:316-328)."""
    return np.max(data, axis=tuple(axes), keepdims=bool(keepdims))


def reduce_min(data, axes, keepdims=1):
    """PureReduceMin: np.min over ``axes`` (pure_implementations.py:331-343)."""
    return np.min(data, axis=tuple(axes), keepdims=bool(keepdims))


def log_softmax(X, axis=-1):
    """PureLogSoftmax, step by step as the reference writes it (pure_implementations.py:594-616):
    max, subtract, exp, sum, log, subtract."""
    reduced_shape = list(X.shape)
    reduced_shape[axis] = 1
    max_keepdims = np.reshape(np.max(X, axis=axis), reduced_shape)
    max_sub = X - max_keepdims
    exp_arr = np.exp(max_sub)
    sum_keepdims = np.reshape(np.sum(exp_arr, axis=axis), reduced_shape)
    log_sum = np.log(sum_keepdims)
    return max_sub - log_sum


def sum_(*inputs):
    """PureSum: all inputs have the output's shape, added left to right (pure_implementations.py:529-591)."""
    out = inputs[0]
    for x in inputs[1:]:
        out = out + x
    return out


def layer_normalization(X, gamma, beta=None, axis=-1, epsilon=1e-5):
    """LayerNormalization as the nine-node chain the reference actually runs
    (there is no LayerNormalization node at opset 12): ReduceMean, Sub, Pow(2),
    ReduceMean, Add(eps), Sqrt, Div, Mul(gamma), Add(beta)
    (pure_implementations.py:97-109, 82-84, 59-74, 77-79, 41-56, 92-94)."""
    axes = list(range(axis % X.ndim, X.ndim))
    mean = reduce_mean(X, axes)                          # ReduceMean
    centred = X - mean                                   # Sub
    squared = centred ** np.asarray(2.0, dtype=X.dtype)  # Pow
    var = reduce_mean(squared, axes)                     # ReduceMean
    var_eps = var + np.asarray(epsilon, dtype=X.dtype)   # Add
    std = np.sqrt(var_eps)                               # Sqrt
    normed = centred / std                               # Div
    out = normed * gamma                                 # Mul
    if beta is not None:
        out = out + beta                                 # Add
    return out.astype(X.dtype, copy=False)


# --------------------------------------------------------------------------- elementwise

try:  # vectorised erf; checked against math.erf in tests/test_oracle.py
    from scipy.special import erf as _erf
except ImportError:  # pragma: no cover
    _erf = np.vectorize(math.erf, otypes=[np.float64])


def erf(X):
    """PureErf (pure_implementations.py:112-127)."""
    return np.asarray(_erf(X)).astype(X.dtype, copy=False)


def gelu(X):
    """Exact Gelu as the exporter's chain Div(sqrt 2), Erf, Add(1), Mul(x), Mul(0.5)
    (each an elementwise map: pure_implementations.py:92-94, 112-127, 77-79, 87-89)."""
    t = X / np.asarray(math.sqrt(2.0), dtype=X.dtype)
    t = erf(t)
    t = t + np.asarray(1.0, dtype=X.dtype)
    t = X * t
    return (t * np.asarray(0.5, dtype=X.dtype)).astype(X.dtype, copy=False)


def relu(X):
    """PureRelu: max(x, 0) in the input dtype (pure_implementations.py:462-474)."""
    return np.maximum(X, np.asarray(0, dtype=X.dtype))


def add(A, B):
    """Add via python_pure_op_implementation (pure_implementations.py:77-79)."""
    return A + B


def sub(A, B):
    return A - B


def mul(A, B):
    return A * B


def div(A, B):
    return A / B


def sqrt(X):
    return np.sqrt(X)


def log(X):
    """PureLog (pure_implementations.py:23-38)."""
    return np.log(X)


def tanh(X):
    """Tanh via python_pure_op_implementation (pure_implementations.py:296-298)."""
    return np.tanh(X)


def reciprocal(X):
    """PureReciprocal: dtype(1) / x (pure_implementations.py:275-293)."""
    return (np.asarray(1, dtype=X.dtype) / X).astype(X.dtype, copy=False)


def softplus(X):
    """Softplus exactly as written in the reference, log(1 + exp(x)), in the input dtype
    (pure_implementations.py:696-698): overflows to inf where exp does."""
    with np.errstate(over="ignore"):
        return np.log(np.asarray(1, dtype=X.dtype) + np.exp(X)).astype(X.dtype, copy=False)


def sigmoid(X):
    """PureSigmoid: dtype(1) / (dtype(1) + exp(-x)) (pure_implementations.py:701-712)."""
    one = np.asarray(1, dtype=X.dtype)
    with np.errstate(over="ignore"):
        return (one / (one + np.exp(-X))).astype(X.dtype, copy=False)


def exp(X):
    """ONNX Exp (no pure expansion in the reference; ONNX Runtime runs it there)."""
    with np.errstate(over="ignore"):
        return np.exp(X)


def neg(X):
    """ONNX Neg (no pure expansion in the reference)."""
    return np.negative(X)


def abs(X):  # noqa: A001 (named after the ONNX op)
    """ONNX Abs (no pure expansion in the reference)."""
    return np.abs(X)


def pow(X, Y):  # noqa: A001 (named after the ONNX op)
    """PurePow (pure_implementations.py:59-74): x ** y, with broadcasting."""
    return np.power(X, np.asarray(Y, dtype=X.dtype)).astype(X.dtype, copy=False)


def maxpool2d(X, kernel_shape, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1)):
    """PureMaxPool2D (img_op_implementations.py:28-161): Y starts at the smallest value and every window element
    is folded in with max. The reference refuses pads and dilations; here padded positions simply do not take
    part (ONNX pads MaxPool with -inf)."""
    N, C, H, W = X.shape
    KH, KW = kernel_shape
    eh, ew = (KH - 1) * dilations[0] + 1, (KW - 1) * dilations[1] + 1
    OH = (H + pads[0] + pads[2] - eh) // strides[0] + 1
    OW = (W + pads[1] + pads[3] - ew) // strides[1] + 1
    Xp = np.full((N, C, H + pads[0] + pads[2], W + pads[1] + pads[3]), -np.inf, dtype=X.dtype)
    Xp[:, :, pads[0]:pads[0] + H, pads[1]:pads[1] + W] = X
    Y = np.full((N, C, OH, OW), -np.inf, dtype=X.dtype)
    for kh in range(KH):
        for kw in range(KW):
            h0, w0 = kh * dilations[0], kw * dilations[1]
            window = Xp[:, :, h0:h0 + (OH - 1) * strides[0] + 1:strides[0], w0:w0 + (OW - 1) * strides[1] + 1:strides[1]]
            Y = np.maximum(Y, window)
    return Y


def global_average_pool(X):
    """GlobalAveragePool (img_op_implementations.py:410-412): mean over axes 2 and 3, kept as size-1 axes."""
    return np.mean(X, axis=tuple(range(2, X.ndim)), keepdims=True).astype(X.dtype, copy=False)


def batch_normalization(X, scale, B, mean, var, epsilon=1e-5):
    """Inference BatchNormalization in the arithmetic order of PureBatchNormalization
    (img_op_implementations.py:362-375), with the stored statistics where the training form uses the batch's:
    (X - mean) * (1 / sqrt(var + eps)) * scale + B, statistics broadcast as [C, 1, ...]."""
    bshape = (1, -1) + (1, ) * (X.ndim - 2)
    one = np.asarray(1.0, dtype=X.dtype)
    normalized = (X - mean.reshape(bshape)) * (one / np.sqrt(var.reshape(bshape) + np.asarray(epsilon, dtype=X.dtype)))
    return (normalized * scale.reshape(bshape) + B.reshape(bshape)).astype(X.dtype, copy=False)


def einsum(equation, *operands):
    """PureEinsum (pure_implementations.py:238-267) lowers to DaCe's einsum SDFG; numpy's einsum is the
    comparator of the reference's own test (tests/pure_expansions/test_expansions.py:456-473)."""
    return np.einsum(equation, *operands)


def cast(X, np_dtype):
    """PureCast (pure_implementations.py:382-430): one map of ``__output = __input``, the C conversion
    (floating point to integer truncates toward zero, as numpy's astype does for values in range)."""
    return X.astype(np_dtype)


def slice_(data, starts, ends, axes=None, steps=None):
    """ONNX Slice; PureSlice (pure_implementations.py:619-693) is the axis-0, step-1 case
    ``data[start:end:1, :]`` with ``end == INT64_MAX`` meaning "to the end". Python slicing already clamps
    bounds the way the operator specifies."""
    axes = list(range(len(starts))) if axes is None else list(axes)
    steps = [1] * len(starts) if steps is None else list(steps)
    index = [slice(None)] * data.ndim
    for s, e, ax, st in zip(starts, ends, axes, steps):
        index[int(ax)] = slice(int(s), int(e), int(st))
    return np.ascontiguousarray(data[tuple(index)])


def transpose(X, perm=None):
    """PureTranspose (pure_implementations.py:369-379)."""
    return np.ascontiguousarray(np.transpose(X, axes=perm))


def reshape(X, shape):
    """PureReshape (pure_implementations.py:477-513)."""
    return np.reshape(X, shape)


# --------------------------------------------------------------------------- BERT encoder layer


def bert_layer_weights(rng, hidden=768, ffn=3072, dtype=np.float32):
    """Seeded weights of the benchmark layer: matrices ~N(0, 0.02) stored [in, out]
    (the layout ONNX MatMul consumes), biases 0, LayerNorm gamma ~N(1, 0.02) and
    beta ~N(0, 0.02). Drawn in a fixed order so every consumer sees the same values."""
    w = {}
    for name, shape in (("wq", (hidden, hidden)), ("wk", (hidden, hidden)), ("wv", (hidden, hidden)),
                        ("wo", (hidden, hidden)), ("w1", (hidden, ffn)), ("w2", (ffn, hidden))):
        w[name] = rng.normal(0.0, 0.02, size=shape).astype(dtype)
    for name, n in (("bq", hidden), ("bk", hidden), ("bv", hidden), ("bo", hidden), ("b1", ffn), ("b2", hidden)):
        w[name] = np.zeros(n, dtype=dtype)
    for i in (1, 2):
        w[f"ln{i}_g"] = rng.normal(1.0, 0.02, size=hidden).astype(dtype)
        w[f"ln{i}_b"] = rng.normal(0.0, 0.02, size=hidden).astype(dtype)
    return w


def bert_layer(x, w, heads=12, eps=1e-12):
    """BERT-base encoder layer (post-LayerNorm, exact Gelu, no mask) composed from
    the op restatements above, node for node as the ONNX graph of the benchmark:
    MatMul, Add, Reshape, Transpose, MatMul, Div, Softmax, MatMul, Transpose,
    Reshape, MatMul, Add, Add, LayerNormalization, MatMul, Add, Gelu, MatMul, Add,
    Add, LayerNormalization. This is the module of tests/pytorch/test_bert_encoder.py:17."""
    bsz, seq, hidden = x.shape
    d = hidden // heads

    def split_heads(t):  # [B,S,H] -> [B,heads,S,d]
        return transpose(reshape(t, (bsz, seq, heads, d)), (0, 2, 1, 3))

    q = split_heads(add(matmul(x, w["wq"]), w["bq"]))
    k = split_heads(add(matmul(x, w["wk"]), w["bk"]))
    v = split_heads(add(matmul(x, w["wv"]), w["bv"]))
    scores = div(matmul(q, transpose(k, (0, 1, 3, 2))), np.asarray(math.sqrt(d), dtype=x.dtype))
    probs = softmax(scores, axis=-1)
    ctx = reshape(transpose(matmul(probs, v), (0, 2, 1, 3)), (bsz, seq, hidden))
    attn = add(matmul(ctx, w["wo"]), w["bo"])
    h1 = layer_normalization(add(attn, x), w["ln1_g"], w["ln1_b"], axis=-1, epsilon=eps)
    inter = gelu(add(matmul(h1, w["w1"]), w["b1"]))
    out = add(matmul(inter, w["w2"]), w["b2"])
    return layer_normalization(add(out, h1), w["ln2_g"], w["ln2_b"], axis=-1, epsilon=eps)

"""Seeded random shapes and attributes for the operators around the contractions -- unary maps, reductions,
LogSoftmax, Cast, Slice, MaxPool, BatchNormalization, GlobalAveragePool, Einsum -- through the node call form,
against the oracle. The fixed cases in test_expansions_gpu.py pin the edge cases; these sweep the space between
them (ranks, ragged extents, negative and out-of-range slice bounds, window geometries that leave partial
windows in the padding). Every seed is printed (and flushed) before its launches."""
import numpy as np
import pytest

import dace_onnx_amd.onnx as donnx
from dace_onnx_amd.onnx import proto
from oracle import pure_ops as O
from conftest import rel_err, FP32_REL_TOL

pytestmark = pytest.mark.gpu

_UNARY = (("Log", ("input", "output"), True), ("Tanh", ("input", "output"), False), ("Exp", ("input", "output"), False),
          ("Sigmoid", ("X", "Y"), False), ("Softplus", ("X", "Y"), False), ("Reciprocal", ("X", "Y"), True),
          ("Neg", ("X", "Y"), False), ("Abs", ("X", "Y"), False))
_EINSUMS = ("bij,jk->bik", "ik,kj->ij", "bhqd,bhkd->bhqk", "bqhd,bkhd->bhqk", "bik,jk->bij", "ij,bjk->bik", "bij,bjk->bki",
            "ijk,jkl->il", "i,j->ij", "bi,bi->b", "abcij,abcjk->abcik", "ij,jk->ki")
_CAST_TYPES = (np.float32, np.int32, np.int64, np.float64, np.int8, np.uint8, np.bool_)


@pytest.mark.parametrize("seed", range(40))
def test_random_operator_cases(seed):
    rng = np.random.default_rng(seed)
    print(f"random operator cases, seed {seed}", flush=True)
    failures = []

    def check(tag, ok):
        if not ok:
            failures.append(tag)

    shape = tuple(int(v) for v in rng.integers(1, 40, size=rng.integers(1, 4)))
    X = rng.normal(scale=3, size=shape).astype(np.float32)
    for op, conns, positive in _UNARY:
        xin = np.abs(X) + np.float32(0.05) if positive else X
        Y = np.zeros_like(X)
        getattr(donnx, "ONNX" + op)(**{conns[0]: xin, conns[1]: Y})
        check(f"{op} {shape}", np.allclose(Y, getattr(O, op.lower())(xin), rtol=3e-6, atol=3e-7))

    shape = tuple(int(v) for v in rng.integers(1, 60, size=rng.integers(1, 5)))
    X = rng.normal(1.0, 2.0, size=shape).astype(np.float32)
    first = int(rng.integers(0, len(shape)))
    axes, keep = list(range(first, int(rng.integers(first, len(shape))) + 1)), int(rng.integers(0, 2))
    for op, oracle in (("ReduceSum", O.reduce_sum), ("ReduceMax", O.reduce_max), ("ReduceMin", O.reduce_min),
                       ("ReduceMean", O.reduce_mean)):
        expected = oracle(X.astype(np.float64), axes, keep)
        Y = np.zeros(expected.shape, np.float32)
        getattr(donnx, "ONNX" + op)(data=X, reduced=Y, axes=axes, keepdims=keep)
        if op in ("ReduceMax", "ReduceMin"):
            check(f"{op} {shape} {axes}", np.array_equal(expected.astype(np.float32), Y))
        else:
            scale = O.reduce_sum(np.abs(X).astype(np.float64), axes, keep) / (1 if op == "ReduceSum" else np.prod([shape[a] for a in axes]))
            check(f"{op} {shape} {axes}", (np.abs(Y - expected) <= 5e-6 * scale + 1e-30).all())
    axis = int(rng.integers(-len(shape), len(shape)))
    Y = np.zeros_like(X)
    donnx.ONNXLogSoftmax(input=X, output=Y, axis=axis)
    check(f"LogSoftmax {shape} {axis}", np.allclose(Y, O.log_softmax(X.astype(np.float64), axis=axis), rtol=1e-5, atol=3e-6))

    src, dst = _CAST_TYPES[rng.integers(0, 7)], _CAST_TYPES[rng.integers(0, 7)]
    n = int(rng.integers(1, 5000))
    Xc = rng.normal(scale=30, size=n) * (rng.random(n) > 0.3)
    Xc = np.abs(Xc).astype(src) if np.uint8 in (src, dst) else Xc.astype(src)     # negative -> unsigned is not defined in C
    Yc = np.zeros(n, dst)
    donnx.ONNXCast(input=Xc, output=Yc, to=proto.np_dtype_to_tensor_dtype(np.dtype(dst)))
    check(f"Cast {src.__name__} -> {dst.__name__} {n}", np.array_equal(O.cast(Xc, dst), Yc))

    shape = tuple(int(v) for v in rng.integers(1, 30, size=rng.integers(1, 5)))
    X = rng.normal(size=shape).astype(np.float32)
    axes = sorted(rng.choice(len(shape), size=int(rng.integers(1, len(shape) + 1)), replace=False).tolist())
    starts = [int(rng.integers(-shape[a] - 2, shape[a] + 2)) for a in axes]
    ends = [int(rng.integers(-shape[a] - 2, shape[a] + 2)) for a in axes]
    steps = [int(rng.choice([1, 1, 2, 3, -1, -2])) for _ in axes]
    expected = O.slice_(X, starts, ends, axes, steps)
    Y = np.full(expected.shape, np.nan, np.float32)
    donnx.ONNXSlice(data=X, output=Y, **{k: np.array(v, np.int64) for k, v in
                                         (("starts", starts), ("ends", ends), ("axes", axes), ("steps", steps))})
    check(f"Slice {shape} {starts} {ends} {axes} {steps}", np.array_equal(expected, Y))

    kh, kw, dh, dw = (int(v) for v in (rng.integers(1, 5), rng.integers(1, 5), rng.integers(1, 3), rng.integers(1, 3)))
    eh, ew = (kh - 1) * dh + 1, (kw - 1) * dw + 1
    pads = [int(rng.integers(0, eh)), int(rng.integers(0, ew)), int(rng.integers(0, eh)), int(rng.integers(0, ew))]
    strides = [int(rng.integers(1, 4)), int(rng.integers(1, 4))]
    X = rng.normal(size=(int(rng.integers(1, 4)), int(rng.integers(1, 9)), int(rng.integers(eh, eh + 30)),
                         int(rng.integers(ew, ew + 30)))).astype(np.float32)
    expected = O.maxpool2d(X, (kh, kw), strides, pads, (dh, dw))
    Y = np.zeros(expected.shape, np.float32)
    donnx.ONNXMaxPool(X=X, Y=Y, kernel_shape=[kh, kw], strides=strides, pads=pads, dilations=[dh, dw])
    check(f"MaxPool {X.shape} k{kh}x{kw} s{strides} p{pads} d{dh},{dw}", np.array_equal(expected, Y))

    C = X.shape[1]
    scale, b, mean = (rng.normal(size=C).astype(np.float32) for _ in range(3))
    var = rng.uniform(0.1, 3.0, size=C).astype(np.float32)
    Z = np.zeros_like(X)
    donnx.ONNXBatchNormalization(X=X, scale=scale, B=b, in_mean=mean, in_var=var, Y=Z, epsilon=1e-5)
    check(f"BatchNormalization {X.shape}", np.allclose(Z, O.batch_normalization(X, scale, b, mean, var, 1e-5), rtol=2e-5, atol=2e-5))
    G = np.zeros(X.shape[:2] + (1, 1), np.float32)
    donnx.ONNXGlobalAveragePool(X=X, Y=G)
    check(f"GlobalAveragePool {X.shape}", np.allclose(G, O.global_average_pool(X.astype(np.float64)), rtol=1e-5, atol=1e-6))

    eq = _EINSUMS[int(rng.integers(0, len(_EINSUMS)))]
    terms = eq.split("->")[0].split(",")
    size = {c: int(rng.integers(1, 24)) for c in set("".join(terms))}
    xs = [rng.normal(size=[size[c] for c in t]).astype(np.float32) for t in terms]
    expected = O.einsum(eq, *[x.astype(np.float64) for x in xs])
    Y = np.zeros(expected.shape, np.float32)
    donnx.ONNXEinsum(Inputs__0=xs[0], Inputs__1=xs[1], Output=Y, equation=eq)
    check(f"Einsum {eq} {size}", rel_err(expected, Y) < FP32_REL_TOL)
    assert not failures, failures

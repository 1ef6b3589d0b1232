"""ctypes loader of ``liboracle_pure.so`` (the C restatement) -- TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "liboracle_pure.so")
_lib = None


def build(force=False):
    if force or not os.path.isfile(_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _PATH


def library():
    global _lib
    if _lib is None:
        if not os.path.isfile(_PATH):
            raise ImportError(f"{_PATH} is not built (run `make -C {_HERE}`)")
        _lib = ctypes.CDLL(_PATH)
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _i64(v):
    return (ctypes.c_int64 * len(v))(*[int(x) for x in v])


def conv2d(X, W, B=None, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1)):
    from .pure_ops import conv_output_shape
    X, W = np.ascontiguousarray(X, np.float32), np.ascontiguousarray(W, np.float32)
    B = None if B is None else np.ascontiguousarray(B, np.float32)
    Y = np.empty(conv_output_shape(X.shape, W.shape, strides, pads, dilations), np.float32)
    n, c, h, w = X.shape
    m, _, kh, kw = W.shape
    library().oracle_conv2d_f32(_p(X), _p(W), _p(B), _p(Y), *[ctypes.c_int64(v) for v in (n, c, h, w, m, kh, kw)],
                                _i64(pads), _i64(strides), _i64(dilations))
    return Y


def softmax(X):
    X = np.ascontiguousarray(X, np.float32)
    Y = np.empty_like(X)
    cols = X.shape[-1]
    library().oracle_softmax_f32(_p(X), _p(Y), ctypes.c_int64(X.size // cols), ctypes.c_int64(cols))
    return Y


def layer_normalization(X, gamma, beta=None, epsilon=1e-5):
    X = np.ascontiguousarray(X, np.float32)
    gamma = np.ascontiguousarray(gamma, np.float32)
    beta = None if beta is None else np.ascontiguousarray(beta, np.float32)
    Y = np.empty_like(X)
    cols = X.shape[-1]
    library().oracle_layernorm_f32(_p(X), _p(gamma), _p(beta), _p(Y), ctypes.c_int64(X.size // cols),
                                   ctypes.c_int64(cols), ctypes.c_float(epsilon))
    return Y


def gelu(X):
    X = np.ascontiguousarray(X, np.float32)
    Y = np.empty_like(X)
    library().oracle_gelu_f32(_p(X), _p(Y), ctypes.c_int64(X.size))
    return Y


def matmul_integer(A, B, a_zero_point=0, b_zero_point=0):
    """int8 / uint8 operands (2-D), zero points scalar, per row of A ([M]) or per column of B ([N])."""
    A, B = np.ascontiguousarray(A), np.ascontiguousarray(B)
    assert A.dtype in (np.int8, np.uint8) and B.dtype in (np.int8, np.uint8) and A.ndim == 2 and B.ndim == 2
    M, K, N = A.shape[0], A.shape[1], B.shape[1]
    za = np.ascontiguousarray(np.asarray(a_zero_point).reshape(-1), np.int32)
    zb = np.ascontiguousarray(np.asarray(b_zero_point).reshape(-1), np.int32)
    assert za.size in (1, M) and zb.size in (1, N)
    Y = np.empty((M, N), np.int32)
    library().oracle_matmul_integer(_p(A), _p(B), _p(za), _p(zb), _p(Y), *[ctypes.c_int64(v) for v in (M, N, K)],
                                    ctypes.c_int(A.dtype == np.uint8), ctypes.c_int(B.dtype == np.uint8),
                                    ctypes.c_int64(0 if za.size == 1 else 1), ctypes.c_int64(0 if zb.size == 1 else 1))
    return Y


def matmul(A, B):
    A, B = np.ascontiguousarray(A, np.float32), np.ascontiguousarray(B, np.float32)
    Y = np.empty((A.shape[0], B.shape[1]), np.float32)
    library().oracle_matmul_f32(_p(A), _p(B), _p(Y), *[ctypes.c_int64(v) for v in (A.shape[0], B.shape[1], A.shape[1])])
    return Y

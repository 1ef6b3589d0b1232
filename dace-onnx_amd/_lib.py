"""ctypes binding of ``libmi355x_onnx.so`` (the C ABI declared in ``include/mi355x_onnx.h``).

The reference loads its own native bridge the same way: a shared library built
ahead of time and opened with ``ctypes.CDLL``
(``daceml/ort_api/raw_api_bindings.py:305-321``), every call checked and turned
into a Python exception (``raw_api_bindings.py:157-162`` raises ``ORTAPIError``).

There is no CPU fallback: if the library is missing or a call returns non-zero
this module raises.
"""
import ctypes
import os
import typing

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_NAME = "libmi355x_onnx.so"
LIBRARY_PATH = os.path.join(_HERE, LIBRARY_NAME)

# status codes / flags, mirrored from include/mi355x_onnx.h
OK = 0
EPI_NONE, EPI_BIAS, EPI_RELU, EPI_GELU, EPI_RESIDUAL, EPI_RELU_AFTER = 0, 1, 2, 4, 8, 16
OP_ADD, OP_SUB, OP_MUL, OP_DIV, OP_POW = 0, 1, 2, 3, 4
OP_RELU, OP_GELU, OP_ERF, OP_SQRT, OP_COPY = 16, 17, 18, 19, 20
REDUCE_MEAN, REDUCE_SUM, REDUCE_MAX, REDUCE_MIN = 0, 1, 2, 3
OP_LOG, OP_TANH, OP_SIGMOID, OP_SOFTPLUS, OP_RECIPROCAL, OP_EXP, OP_NEG, OP_ABS = 21, 22, 23, 24, 25, 26, 27, 28
PROGRAM_REG, PROGRAM_TENSOR, PROGRAM_VECTOR, PROGRAM_IMMEDIATE = 0, 1, 2, 3
PROGRAM_MAX_INSTR, PROGRAM_MAX_TENSORS, PROGRAM_MAX_VECTORS, PROGRAM_MAX_IMM = 16, 4, 4, 8

_c_i64_p = ctypes.POINTER(ctypes.c_int64)
_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float

#: every symbol of the C ABI with (restype, argtypes); tests check that the
#: built library exports exactly these
SIGNATURES: typing.Dict[str, typing.Tuple[typing.Any, typing.List[typing.Any]]] = {
    "mi355x_version": (_int, []),
    "mi355x_last_error": (ctypes.c_char_p, []),
    "mi355x_device_cu_count": (_int, []),
    "mi355x_reload_tuning": (None, []),
    "mi355x_launch_empty_kernel": (_int, [_vp]),
    "mi355x_gemm_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                               _c_i64_p, _c_i64_p, _c_i64_p, _c_i64_p, _f32, _int, _vp]),
    "mi355x_conv2d_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                 _c_i64_p, _c_i64_p, _c_i64_p, _int, _vp]),
    "mi355x_conv2d_res_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                     _c_i64_p, _c_i64_p, _c_i64_p, _int, _vp]),
    "mi355x_matmul_integer": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _i64, _i64, _vp]),
    "mi355x_matmul_integer_i8": (_int, [_vp, _vp, _vp, _vp, _vp,
                                        _i64, _i64, _i64, _vp]),
    "mi355x_softmax_f32": (_int, [_vp, _vp, _i64, _i64, _i64, _vp]),
    "mi355x_attention_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                    _c_i64_p, _c_i64_p, _c_i64_p, _c_i64_p, _f32, _vp]),
    "mi355x_layernorm_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _f32, _vp]),
    "mi355x_reduce_mean_f32": (_int, [_vp, _vp, _i64, _i64, _i64, _vp]),
    "mi355x_maxpool2d_f32": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _c_i64_p, _c_i64_p, _c_i64_p, _vp]),
    "mi355x_batchnorm_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _vp]),
    "mi355x_cast": (_int, [_vp, _int, _vp, _int, _i64, _vp]),
    "mi355x_reduce_f32": (_int, [_int, _vp, _vp, _i64, _i64, _i64, _vp]),
    "mi355x_reduce_nd_f32": (_int, [_int, _vp, _vp, _int, _c_i64_p, _c_i64_p, _c_i64_p, _vp]),
    "mi355x_log_softmax_f32": (_int, [_vp, _vp, _i64, _i64, _i64, _vp]),
    "mi355x_eltwise_f32": (_int, [_int, _vp, _vp, _vp, _int, _c_i64_p, _c_i64_p, _c_i64_p, _vp]),
    "mi355x_permute_b32": (_int, [_vp, _vp, _int, _c_i64_p, _c_i64_p, _vp]),
    "mi355x_eltwise_program_f32": (_int, [ctypes.POINTER(ctypes.c_void_p), _int, ctypes.POINTER(ctypes.c_void_p), _int, _vp,
                                          _i64, _i64, ctypes.POINTER(ctypes.c_uint32), _int,
                                          ctypes.POINTER(ctypes.c_float), _int, _vp]),
}


class MI355XError(RuntimeError):
    """A call into libmi355x_onnx.so returned a non-zero status."""


class LibraryNotBuilt(ImportError):
    """libmi355x_onnx.so is missing: run ``__graft_entry__.build()`` (or ``make`` in csrc/)."""


_lib = None


def library() -> ctypes.CDLL:
    """Open (once) and return the shared library, with prototypes attached."""
    global _lib
    if _lib is None:
        if not os.path.isfile(LIBRARY_PATH):
            raise LibraryNotBuilt(
                f"{LIBRARY_PATH} not found; build it with `python -c 'import __graft_entry__ as g; "
                f"g.build()'` or `make -C {os.path.join(_HERE, 'csrc')}`")
        lib = ctypes.CDLL(LIBRARY_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    if status != OK:
        msg = library().mi355x_last_error().decode("utf-8", "replace")
        raise MI355XError(f"{what} failed with status {status}: {msg}")


def i64_array(values: typing.Sequence[int]):
    return (ctypes.c_int64 * len(values))(*[int(v) for v in values])


def u32_array(values: typing.Sequence[int]):
    return (ctypes.c_uint32 * max(len(values), 1))(*[int(v) for v in values])


def f32_array(values: typing.Sequence[float]):
    return (ctypes.c_float * max(len(values), 1))(*[float(v) for v in values])


def pointer_array(addresses: typing.Sequence[int]):
    return (ctypes.c_void_p * max(len(addresses), 1))(*[int(a) for a in addresses])


def current_stream() -> int:
    """The hipStream_t kernels are enqueued on: torch's current stream."""
    import torch
    return torch.cuda.current_stream().cuda_stream


def ptr(t) -> typing.Optional[int]:
    """Device pointer of a torch tensor (None passes NULL)."""
    return None if t is None else t.data_ptr()

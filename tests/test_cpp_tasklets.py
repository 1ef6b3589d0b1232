"""The second caller of the C ABI: C++ tasklets. An expansion's ``KernelCall.as_cpp()`` is the body DaCe would
compile into the SDFG's library (``cudnn_implementations.py:324-334`` is the reference's template for such a
tasklet, ``environments/cudnn.py:11-67`` for the environment that supplies header and library). ``dace`` is not
installed here, so the code DaCe would emit around the tasklets comes from ``CompiledSDFG.program_source()``;
these tests compile it with the host compiler against ``include/mi355x_onnx.h``, link it with
``libmi355x_onnx.so`` and run it.
"""
import ctypes
import os
import subprocess

import numpy as np
import pytest

import dace_onnx_amd.onnx as donnx
from dace_onnx_amd.onnx import proto
from dace_onnx_amd import sdfg as dace
from dace_onnx_amd.testing.graphs import bert_encoder_layer_model
from dace_onnx_amd.util import utils
from oracle import pure_ops as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBDIR = os.path.join(ROOT, "dace-onnx_amd")
FP32_REL_TOL = 1e-4


def rel_err(expected, got):
    expected = np.asarray(expected, np.float64)
    return float(np.abs(np.asarray(got, np.float64) - expected).max() / max(np.abs(expected).max(), 1e-30))


def _build(source, name, directory, syntax_only=False):
    path = os.path.join(directory, name + ".cpp")
    with open(path, "w") as f:
        f.write(source)
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include")]
    if syntax_only:
        subprocess.run(cmd + ["-fsyntax-only", path], check=True, capture_output=True, text=True)
        return None
    out = os.path.join(directory, f"lib{name}.so")
    subprocess.run(cmd + ["-shared", "-fPIC", path, "-o", out, "-L", LIBDIR, "-lmi355x_onnx", f"-Wl,-rpath,{LIBDIR}"],
                   check=True, capture_output=True, text=True)
    return out


def _small_bert():
    w = O.bert_layer_weights(np.random.default_rng(5), hidden=128, ffn=256)
    for k in ("bq", "bk", "bv", "bo", "b1", "b2"):   # non-zero biases: every epilogue operand matters
        w[k] = np.random.default_rng(6).normal(0, 0.02, size=w[k].shape).astype(np.float32)
    return w, donnx.ONNXModel("bert_cpp", bert_encoder_layer_model(w, 2, 128, 2))


def _single_node(node, inputs, outputs):
    sdfg = dace.SDFG(node.label)
    st = sdfg.add_state()
    st.add_node(node)
    for conn, (shape, dtype) in inputs.items():
        sdfg.add_array(conn + "_in", shape, dtype)
        node.add_in_connector(conn)
        st.add_edge(st.add_read(conn + "_in"), None, node, conn, sdfg.make_array_memlet(conn + "_in"))
    for conn, (shape, dtype) in outputs.items():
        sdfg.add_array(conn + "_out", shape, dtype)
        node.add_out_connector(conn)
        st.add_edge(node, conn, st.add_write(conn + "_out"), None, sdfg.make_array_memlet(conn + "_out"))
    utils.expand_onnx_nodes(sdfg)
    return sdfg


def _conv_sdfg():
    return _single_node(donnx.ONNXConv("conv_cpp", strides=[2, 2], pads=[1, 1, 1, 1]),
                        {"X": ([2, 8, 12, 12], dace.float32), "W": ([16, 8, 3, 3], dace.float32), "B": ([16], dace.float32)},
                        {"Y": ([2, 16, 6, 6], dace.float32)})


def _mmi_sdfg():
    return _single_node(donnx.ONNXMatMulInteger("mmi_cpp"),
                        {"A": ([64, 128], dace.uint8), "B": ([128, 48], dace.int8), "a_zero_point": ([64], dace.uint8),
                         "b_zero_point": ([1], dace.int8)}, {"Y": ([64, 48], dace.int32)})


def test_generated_program_compiles_against_the_header(tmp_path):
    """No GPU needed: the tasklet text of the fused BERT layer, of a Conv and of a MatMulInteger is valid C++
    against the C ABI's header (warnings are errors), one tasklet per launch."""
    _, model = _small_bert()
    compiled = dace.CompiledSDFG(model.expand())
    source, arrays = compiled.program_source("bert_cpp")
    assert source.count("int __status = mi355x_") == compiled.num_launches == 7
    assert "__dace_current_stream" in source and '#include "mi355x_onnx.h"' in source
    assert arrays[:len(compiled._external)] == compiled._external
    _build(source, "bert_cpp", str(tmp_path), syntax_only=True)
    for make in (_conv_sdfg, _mmi_sdfg):
        sdfg = make()
        source, _ = dace.CompiledSDFG(sdfg).program_source()
        _build(source, sdfg.name, str(tmp_path), syntax_only=True)


def test_integer_view_keeps_its_element_type(tmp_path):
    """A Reshape of an int32 result is a view (no launch); the tasklet that reads it declares the view with the
    view's own element type, not as float*."""
    H, T = proto.helper, proto.TensorProto
    nodes = [H.make_node("MatMulInteger", ["a", "b"], ["y"]), H.make_node("Reshape", ["y", "shape"], ["yr"]),
             H.make_node("Cast", ["yr"], ["out"], to=1)]
    g = H.make_graph(nodes, "g", [H.make_tensor_value_info("a", T.INT8, [64, 128]), H.make_tensor_value_info("b", T.INT8, [128, 48])],
                     [H.make_tensor_value_info("out", T.FLOAT, [48, 64])],
                     initializer=[proto.numpy_helper.from_array(np.array([48, 64], np.int64), "shape")])
    model = donnx.ONNXModel("intview", H.make_model(g, opset_imports=[H.make_opsetid("", 12)]))
    source, _ = dace.CompiledSDFG(model.expand()).program_source("intview")
    assert "// yr is a view of y" in source
    cast = source[source.index("// Cast"):]
    assert "int32_t* _input = (int32_t*)" in cast and "float* _input" not in cast
    _build(source, "intview", str(tmp_path), syntax_only=True)


def _run_program(compiled, name, tensors, tmp_path):
    """Compile and call __program_<name>; ``tensors`` maps array name / key to a torch tensor, transients that
    are missing are allocated here."""
    import torch
    source, arrays = compiled.program_source(name)
    lib = ctypes.CDLL(_build(source, name, str(tmp_path)))
    fn = getattr(lib, "__program_" + name)
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p]
    transients = compiled.transient_descriptors()
    held = dict(tensors)
    for key in arrays:
        if key not in held:
            d = transients[key]
            held[key] = torch.full(tuple(d.shape), 0, dtype=d.dtype.as_torch(), device="cuda")
    table = (ctypes.c_void_p * len(arrays))(*[held[k].data_ptr() for k in arrays])
    stream = torch.cuda.current_stream().cuda_stream
    assert fn(table, ctypes.c_void_p(stream)) == 0
    torch.cuda.synchronize()
    return held


@pytest.mark.gpu
def test_generated_program_runs_the_bert_layer(tmp_path):
    import torch
    w, model = _small_bert()
    x = np.random.default_rng(7).normal(size=(2, 128, 128)).astype(np.float32)
    expected = O.bert_layer(x, w, heads=2)
    y_ctypes = model(torch.from_numpy(x).cuda())          # first caller: ctypes
    compiled = model.compile_and_init()
    tensors = {"x": torch.from_numpy(x).cuda(), "y": torch.full((2, 128, 128), float("nan"), device="cuda"), **model.clean_weights}
    held = _run_program(compiled, "bert_cpp", tensors, tmp_path)   # second caller: compiled C++ tasklets
    got = held["y"].cpu().numpy()
    assert rel_err(expected, got) < FP32_REL_TOL
    assert np.array_equal(got, y_ctypes.cpu().numpy())     # the same launches with the same arguments


@pytest.mark.gpu
def test_generated_program_runs_conv_and_matmul_integer(tmp_path):
    import torch
    rng = np.random.default_rng(8)
    X = rng.normal(size=(2, 8, 12, 12)).astype(np.float32)
    W = rng.normal(size=(16, 8, 3, 3)).astype(np.float32)
    B = rng.normal(size=16).astype(np.float32)
    compiled = dace.CompiledSDFG(_conv_sdfg())
    held = _run_program(compiled, "conv_cpp", {"X_in": torch.from_numpy(X).cuda(), "W_in": torch.from_numpy(W).cuda(),
                                               "B_in": torch.from_numpy(B).cuda(),
                                               "Y_out": torch.full((2, 16, 6, 6), float("nan"), device="cuda")}, tmp_path)
    assert rel_err(O.conv2d(X, W, B, (2, 2), (1, 1, 1, 1)), held["Y_out"].cpu().numpy()) < FP32_REL_TOL

    A = rng.integers(0, 256, size=(64, 128)).astype(np.uint8)
    Bm = rng.integers(-128, 128, size=(128, 48), dtype=np.int8)
    za = rng.integers(0, 256, size=64).astype(np.uint8)
    zb = np.array([-5], np.int8)
    compiled = dace.CompiledSDFG(_mmi_sdfg())
    held = _run_program(compiled, "mmi_cpp", {"A_in": torch.from_numpy(A).cuda(), "B_in": torch.from_numpy(Bm).cuda(),
                                              "a_zero_point_in": torch.from_numpy(za).cuda(),
                                              "b_zero_point_in": torch.from_numpy(zb).cuda(),
                                              "Y_out": torch.full((64, 48), -1, dtype=torch.int32, device="cuda")}, tmp_path)
    assert np.array_equal(O.matmul_integer(A, Bm, za, zb), held["Y_out"].cpu().numpy())   # bit-exact

"""The benchmark configurations at full size, the committed golden fixtures, and
ONNXModel end to end -- all through the C ABI on the GPU.

Full-size expectations come from the oracle where it finishes in seconds (its C
restatement for the convolution and the integer product) and from
size-independent properties otherwise.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from dace_onnx_amd import _lib, sdfg as dace
import dace_onnx_amd.onnx as donnx
from dace_onnx_amd.testing.graphs import bert_encoder_layer_model, conv_relu_model
from dace_onnx_amd.onnx import proto
from oracle import pure_ops as O
from conftest import rel_err, FP32_REL_TOL, GOLDEN_DIR

pytestmark = pytest.mark.gpu


# ----------------------------------------------------------------------------- golden fixtures
def test_golden_fixtures_through_hip(golden):
    Y = np.zeros_like(golden["conv1_Y"])
    donnx.ONNXConv(X=golden["conv1_X"], W=golden["conv1_W"], Y=Y, strides=[2, 2])
    assert rel_err(golden["conv1_Y"], Y) < FP32_REL_TOL

    Y = np.zeros_like(golden["softmax_Y"])
    donnx.ONNXSoftmax(input=golden["softmax_X"], output=Y, axis=-1)
    assert rel_err(golden["softmax_Y"], Y) < FP32_REL_TOL

    Y = np.zeros_like(golden["ln_Y"])
    donnx.ONNXLayerNormalization(X=golden["ln_X"], Scale=golden["ln_gamma"], B=golden["ln_beta"], Y=Y, axis=-1,
                                 epsilon=1e-12)
    assert rel_err(golden["ln_Y"], Y) < FP32_REL_TOL

    Y = np.zeros_like(golden["gelu_Y"])
    donnx.ONNXGelu(X=golden["gelu_X"], Y=Y)
    assert rel_err(golden["gelu_Y"], Y) < FP32_REL_TOL

    Y = np.zeros_like(golden["matmul_Y"])
    donnx.ONNXMatMul(A=golden["matmul_A"], B=golden["matmul_B"], Y=Y)
    assert rel_err(golden["matmul_Y"], Y) < FP32_REL_TOL

    Y = np.zeros_like(golden["gemm_Y"])
    donnx.ONNXGemm(A=golden["gemm_A"], B=golden["gemm_B"], C=golden["gemm_C"], Y=Y, transB=1)
    assert rel_err(golden["gemm_Y"], Y) < FP32_REL_TOL

    Y = np.zeros_like(golden["mmi_Y"])
    donnx.ONNXMatMulInteger(A=golden["mmi_A"], B=golden["mmi_B"], a_zero_point=np.array(3, np.int8),
                            b_zero_point=np.array(-2, np.int8), Y=Y)
    assert np.array_equal(golden["mmi_Y"], Y)


def test_golden_conv_relu_model(golden):
    m = conv_relu_model(golden["conv2_W"], golden["conv2_B"], golden["conv2_X"].shape, pads=(1, 2, 0, 1), strides=(2, 1))
    m.graph.node[0].attribute.append(proto.AttributeProto("dilations", [1, 2]))
    for fuse in (False, True):
        got = donnx.ONNXModel("conv_relu", proto.parse_model(proto.serialize_model(m)), fuse=fuse)(golden["conv2_X"])
        assert rel_err(golden["conv2_Y"], got) < FP32_REL_TOL


@pytest.mark.parametrize("fuse", [False, True])
def test_golden_bert_layer_model(golden, fuse):
    hidden, heads, ffn, bsz, seq = (int(v) for v in golden["bert_meta"])
    w = {k[len("bert_"):]: golden[k] for k in golden.files if k.startswith("bert_") and k not in
         ("bert_x", "bert_y", "bert_meta")}
    model = donnx.ONNXModel("bert_small", bert_encoder_layer_model(w, bsz, seq, heads), fuse=fuse)
    got = model(golden["bert_x"])
    assert rel_err(golden["bert_y"], got) < FP32_REL_TOL
    # the model also runs from its serialized .onnx form and on torch tensors
    m2 = donnx.ONNXModel("bert_small_file", proto.serialize_model(bert_encoder_layer_model(w, bsz, seq, heads)), fuse=fuse)
    got2 = m2(x=torch.from_numpy(golden["bert_x"]).cuda())
    assert isinstance(got2, torch.Tensor) and got2.is_cuda
    assert np.array_equal(got, got2.cpu().numpy())


@pytest.mark.parametrize("fuse", [False, True])
def test_golden_bert_layer_in_exported_opset12_form(golden, fuse):
    # LayerNorm and Gelu spelled out as the exporter writes them below opset 17 (what the reference runs)
    hidden, heads, ffn, bsz, seq = (int(v) for v in golden["bert_meta"])
    w = {k[len("bert_"):]: golden[k] for k in golden.files if k.startswith("bert_") and k not in
         ("bert_x", "bert_y", "bert_meta")}
    model = donnx.ONNXModel("bert_small_op12", bert_encoder_layer_model(w, bsz, seq, heads, decomposed=True), fuse=fuse)
    got = model(golden["bert_x"])
    assert model.compile_and_init().num_launches == (9 if fuse else 46)
    assert rel_err(golden["bert_y"], got) < FP32_REL_TOL


def test_matmuls_sharing_an_input_are_fused_into_one_wide_gemm():
    # y1 = x w1 + b1 and y2 = x w2 + b2 become one GEMM; their readers address column slices of its result
    rng = np.random.default_rng(7)
    x = rng.normal(size=(3, 20, 32)).astype(np.float32)
    w1, w2 = rng.normal(size=(32, 24)).astype(np.float32), rng.normal(size=(32, 8)).astype(np.float32)
    b1, b2 = rng.normal(size=24).astype(np.float32), rng.normal(size=8).astype(np.float32)
    w3, w4 = rng.normal(size=(24, 12)).astype(np.float32), rng.normal(size=(40, 20)).astype(np.float32)
    H = proto.helper
    nodes = [H.make_node("MatMul", ["x", "w1"], ["y1m"]), H.make_node("Add", ["y1m", "b1"], ["y1"]),
             H.make_node("MatMul", ["x", "w2"], ["y2m"]), H.make_node("Add", ["b2", "y2m"], ["y2"]),
             H.make_node("MatMul", ["y1", "w3"], ["z1"]), H.make_node("MatMul", ["w4", "y2"], ["z2"])]
    g = H.make_graph(nodes, "g", [H.make_tensor_value_info("x", 1, list(x.shape))],
                     [H.make_tensor_value_info("z1", 1, None), H.make_tensor_value_info("z2", 1, None)],
                     initializer=[proto.numpy_helper.from_array(a, n) for a, n in
                                  ((w1, "w1"), (w2, "w2"), (b1, "b1"), (b2, "b2"), (w3, "w3"), (w4, "w4"))])
    x64 = x.astype(np.float64)
    want1 = (x64 @ w1 + b1) @ w3
    want2 = w4.astype(np.float64) @ (x64 @ w2 + b2)
    for fuse in (False, True):
        model = donnx.ONNXModel(f"hfuse_{fuse}", H.make_model(g), fuse=fuse)
        z1, z2 = model(x)
        assert model.compile_and_init().num_launches == (3 if fuse else 6)
        assert rel_err(want1, z1) < FP32_REL_TOL and rel_err(want2, z2) < FP32_REL_TOL


# ----------------------------------------------------------------------------- config 2: softmax / layernorm
def test_config2_softmax_full_size():
    X = np.random.default_rng(2).normal(size=(8, 12, 128, 128)).astype(np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXSoftmax(input=X, output=Y, axis=-1)
    expected = O.softmax(X)
    assert rel_err(expected, Y) < FP32_REL_TOL
    # element by element as well, so that probabilities down to 1e-6 are held to 1e-4 of their own size
    # (the closeness rule of the reference's tests, daceml/testing/utils.py:6)
    assert np.allclose(expected, Y, rtol=1e-4, atol=1e-6)
    assert np.abs(Y.sum(-1) - 1.0).max() < 1e-5


def test_config2_layernorm_full_size():
    rng = np.random.default_rng(2)
    rng.normal(size=(8, 12, 128, 128))  # tensors of one config are drawn in the order listed
    X = rng.normal(size=(8, 128, 768)).astype(np.float32)
    g = rng.normal(1.0, 0.02, size=768).astype(np.float32)
    b = rng.normal(0.0, 0.02, size=768).astype(np.float32)
    Y = np.zeros_like(X)
    donnx.ONNXLayerNormalization(X=X, Scale=g, B=b, Y=Y, axis=-1, epsilon=1e-12)
    expected = O.layer_normalization(X, g, b, epsilon=1e-12)
    assert rel_err(expected, Y) < FP32_REL_TOL
    # element by element: outputs near zero are held to an absolute 1e-5, the rest to 1e-4 of their own size
    assert np.allclose(expected, Y, rtol=1e-4, atol=1e-5)


# ----------------------------------------------------------------------------- config 3: BERT-base encoder layer
@pytest.fixture(scope="module")
def bert_case():
    rng = np.random.default_rng(3)
    w = O.bert_layer_weights(rng)
    x = rng.normal(size=(8, 128, 768)).astype(np.float32)
    return w, x, O.bert_layer(x, w, heads=12)


@pytest.mark.parametrize("fuse", [False, True])
def test_config3_bert_layer(bert_case, fuse):
    w, x, expected = bert_case
    model = donnx.ONNXModel("bert_base_layer", bert_encoder_layer_model(w, 8, 128, 12), fuse=fuse)
    got = model(x)
    assert got.shape == (8, 128, 768)
    assert rel_err(expected, got) < FP32_REL_TOL
    # the reference's own closeness bar for this module (daceml/testing/utils.py:6)
    assert torch.allclose(torch.from_numpy(expected), torch.from_numpy(got), rtol=1e-4, atol=1e-4)
    # every node ran as a kernel of the library; nothing was left to a fallback
    assert not any(isinstance(n, dace.LibraryNode) for n, _ in model.sdfg.all_nodes_recursive())


def test_config3_hip_graph_replays_match_eager(bert_case):
    w, x, expected = bert_case
    model = donnx.ONNXModel("bert_graph", bert_encoder_layer_model(w, 8, 128, 12), use_hip_graph=True)
    xt = torch.from_numpy(x).cuda()
    eager = model(xt).clone()  # first call runs eagerly and captures
    rng = np.random.default_rng(33)
    for i in range(4):
        xi = torch.from_numpy(rng.normal(size=x.shape).astype(np.float32)).cuda() if i % 2 else xt
        replayed = model(xi)
        torch.cuda.synchronize()
        # eager work and synchronisation between replays, every replay checked
        ref = donnx.ONNXModel(f"bert_eager_{i}", bert_encoder_layer_model(w, 8, 128, 12))(xi)
        assert torch.equal(replayed, ref)
    assert rel_err(expected, eager.cpu().numpy()) < FP32_REL_TOL


# ----------------------------------------------------------------------------- config 4: ResNet Conv + Relu
def test_config4_conv_relu_full_size(c_oracle, tuning):
    rng = np.random.default_rng(4)
    X = rng.normal(size=(32, 64, 56, 56)).astype(np.float32)
    W = (rng.normal(size=(64, 64, 3, 3)) * np.sqrt(2.0 / 576)).astype(np.float32)
    B = np.zeros(64, np.float32)
    model = donnx.ONNXModel("resnet_conv", conv_relu_model(W, B, X.shape))
    Y = model(X)
    assert Y.shape == (32, 64, 56, 56)
    # oracle (C restatement) on a batch slice that finishes in seconds ...
    expected = O.relu(c_oracle.conv2d(X[:4], W, B, (1, 1), (1, 1, 1, 1), (1, 1)))
    assert rel_err(expected, Y[:4]) < FP32_REL_TOL
    # ... and the whole tensor against the reference's comparator (test_conv_expansion.py:30-35)
    full = torch.relu(torch.nn.functional.conv2d(torch.from_numpy(X), torch.from_numpy(W), torch.from_numpy(B),
                                                 padding=1)).numpy()
    assert rel_err(full, Y) < FP32_REL_TOL
    # element by element (tests/pure_expansions/test_conv_expansion.py compares with allclose as well)
    assert np.allclose(expected, Y[:4], rtol=1e-4, atol=1e-5)
    assert np.allclose(full, Y, rtol=1e-4, atol=1e-5)
    # size-independent property: linearity of the convolution before the Relu
    Y1, Y2 = np.zeros_like(Y), np.zeros_like(Y)
    donnx.ONNXConv(X=X, W=W, Y=Y1, pads=[1, 1, 1, 1])
    donnx.ONNXConv(X=(2 * X).astype(np.float32), W=W, Y=Y2, pads=[1, 1, 1, 1])
    assert rel_err(2 * Y1, Y2) < 1e-6
    assert np.array_equal(np.maximum(Y1, 0), Y)
    # the six-deep register ring (two workgroups per CU) in place of the lean kernel the library takes: same bits
    tuning(MI355X_CONV_PER_CU=2)
    Y3 = np.zeros_like(Y)
    donnx.ONNXConv(X=X, W=W, Y=Y3, pads=[1, 1, 1, 1])
    assert np.array_equal(Y1, Y3)


# ----------------------------------------------------------------------------- config 5: MatMulInteger
def test_config5_matmul_integer_full_size(c_oracle):
    rng = np.random.default_rng(5)
    A = rng.integers(-128, 128, size=(4096, 768), dtype=np.int8)
    B = rng.integers(-128, 128, size=(768, 3072), dtype=np.int8)
    Y = np.zeros((4096, 3072), np.int32)
    donnx.ONNXMatMulInteger(A=A, B=B, a_zero_point=np.array(3, np.int8), b_zero_point=np.array(-2, np.int8), Y=Y)
    assert np.array_equal(c_oracle.matmul_integer(A, B, 3, -2), Y)  # bit-exact, every element
    # checksum of checksums: sum_mn Y = (colsum_A - M*za) . (rowsum_B - N*zb)
    ca = A.astype(np.int64).sum(0) - 3 * 4096
    rb = B.astype(np.int64).sum(1) + 2 * 3072
    assert int(Y.astype(np.int64).sum()) == int(ca @ rb)


# ----------------------------------------------------------------------------- C ABI called directly
def test_c_abi_direct_call_and_error_status():
    lib = _lib.library()
    assert lib.mi355x_device_cu_count() == 256
    x = torch.randn(512, 128, device="cuda")
    y = torch.empty_like(x)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        status = lib.mi355x_softmax_f32(x.data_ptr(), y.data_ptr(), 512, 128, 1, stream.cuda_stream)
    assert status == 0
    stream.synchronize()
    assert rel_err(O.softmax(x.cpu().numpy()), y.cpu().numpy()) < FP32_REL_TOL
    # a bad call launches nothing and reports why
    bad = lib.mi355x_conv2d_f32(x.data_ptr(), x.data_ptr(), None, y.data_ptr(), 1, 1, 4, 4, 1, 9, 9,
                                _lib.i64_array([0, 0, 0, 0]), _lib.i64_array([1, 1]), _lib.i64_array([1, 1]), 0, None)
    assert bad == 1 and b"kernel larger than padded input" in lib.mi355x_last_error()


def test_strided_gemm_head_split_merge_without_copies():
    """Q/K/V head split and the context merge expressed as strides of one GEMM call."""
    lib = _lib.library()
    rng = np.random.default_rng(6)
    B_, S, Hh, D = 8, 128, 12, 64
    q = torch.from_numpy(rng.normal(size=(B_, S, Hh * D)).astype(np.float32)).cuda()
    k = torch.from_numpy(rng.normal(size=(B_, S, Hh * D)).astype(np.float32)).cuda()
    scores = torch.empty(B_, Hh, S, S, device="cuda")
    st = _lib.current_stream()
    a_str = _lib.i64_array([S * Hh * D, D, Hh * D, 1])   # [b, h, s, d] view of [B,S,H*D]
    b_str = _lib.i64_array([S * Hh * D, D, 1, Hh * D])   # K^T: [b, h, d, s]
    c_str = _lib.i64_array([Hh * S * S, S * S, S])
    _lib.check(lib.mi355x_gemm_f32(q.data_ptr(), k.data_ptr(), scores.data_ptr(), None, None, B_, Hh, S, S, D,
                                   a_str, b_str, c_str, None, 0.125, 0, st), "gemm")
    qh = q.view(B_, S, Hh, D).permute(0, 2, 1, 3).double()
    kh = k.view(B_, S, Hh, D).permute(0, 2, 1, 3).double()
    ref = 0.125 * (qh @ kh.transpose(2, 3))
    assert rel_err(ref.cpu().numpy(), scores.cpu().numpy()) < FP32_REL_TOL
    # context written straight into the merged [B,S,H*D] layout
    v = torch.from_numpy(rng.normal(size=(B_, S, Hh * D)).astype(np.float32)).cuda()
    probs = torch.softmax(scores, -1)
    ctx = torch.empty(B_, S, Hh * D, device="cuda")
    _lib.check(lib.mi355x_gemm_f32(probs.data_ptr(), v.data_ptr(), ctx.data_ptr(), None, None, B_, Hh, S, D, S,
                                   _lib.i64_array([Hh * S * S, S * S, S, 1]), _lib.i64_array([S * Hh * D, D, Hh * D, 1]),
                                   _lib.i64_array([S * Hh * D, D, Hh * D]), None, 1.0, 0, st), "gemm")
    vh = v.view(B_, S, Hh, D).permute(0, 2, 1, 3).double()
    ref = (probs.double() @ vh).permute(0, 2, 1, 3).reshape(B_, S, Hh * D)
    assert rel_err(ref.cpu().numpy(), ctx.cpu().numpy()) < FP32_REL_TOL


# ----------------------------------------------------------------------------- GEMM kernel variants, ragged shapes
@pytest.mark.parametrize("tile", ["auto", "48", "48x3", "48x2", "48w16", "64", "96", "96w8", "144", "128x48", "128x48x3", "ksplit"])
@pytest.mark.parametrize("M, N, K, epi", [(64, 48, 32, 0), (1, 4, 32, 1), (130, 52, 64, 9), (257, 100, 96, 5), (200, 148, 160, 3),
                                          (1024, 768, 768, 9), (63, 764, 224, 8), (100, 52, 2112, 9)])   # last: 64-k tiles
def test_k_contiguous_gemm_tiles_and_epilogues(tuning, tile, M, N, K, epi):
    """Both operands k-contiguous (activations x [N, K] weights): every tile variant of that kernel on shapes that
    leave partial tiles in M and N, with each epilogue combination (1 bias, 2 relu, 4 gelu, 8 residual) and alpha."""
    if tile == "ksplit":   # 32 x 96 tiles, the eight waves of a workgroup split K (K = 32 and 64: some waves get no slice)
        tuning(MI355X_GEMM_KSPLIT=1)
    elif tile == "128x48":
        tuning(MI355X_GEMM_NT_BM=128, MI355X_GEMM_NT_BN=48, MI355X_GEMM_NT_PER_CU=2)
    elif tile == "128x48x3":
        tuning(MI355X_GEMM_NT_BM=128, MI355X_GEMM_NT_BN=48, MI355X_GEMM_NT_PER_CU=3)
    elif tile == "96w8":    # 128 x 96 tiles by eight waves (the library runs them as 16: 8 wave rows x 2 k-split groups)
        tuning(MI355X_GEMM_NT_BN=96, MI355X_GEMM_NT_WAVES=8)
    elif tile == "48w16":   # 64 x 48 tiles by 16 waves, four k-split groups (where K is a multiple of 64; eight waves elsewhere)
        tuning(MI355X_GEMM_NT_BN=48, MI355X_GEMM_NT_WAVES=16)
    elif tile in ("48x3", "48x2"):   # 64 x 48 tiles as the lean kernel (three workgroups per CU) and as the 64-k one, whatever K
        tuning(MI355X_GEMM_NT_BN=48, MI355X_GEMM_NT_PER_CU=tile[-1])
    else:
        tuning(MI355X_GEMM_NT_BN=None if tile == "auto" else tile)   # the variables are read once; the fixture reloads them
    lib = _lib.library()
    rng = np.random.default_rng(M * 7 + N * 3 + K + epi)
    a = torch.from_numpy(rng.normal(size=(2, M, K)).astype(np.float32)).cuda()
    w = torch.from_numpy(rng.normal(size=(N, K)).astype(np.float32)).cuda()          # [N, K]: B[k, n] = w[n, k]
    bias = torch.from_numpy(rng.normal(size=N).astype(np.float32)).cuda()
    res = torch.from_numpy(rng.normal(size=(2, M, N)).astype(np.float32)).cuda()
    out = torch.full((2, M, N), float("nan"), device="cuda")
    alpha = 0.5
    _lib.check(lib.mi355x_gemm_f32(a.data_ptr(), w.data_ptr(), out.data_ptr(), bias.data_ptr(), res.data_ptr(), 1, 2, M, N, K,
                                   _lib.i64_array([0, M * K, K, 1]), _lib.i64_array([0, 0, 1, K]), _lib.i64_array([0, M * N, N]),
                                   _lib.i64_array([0, M * N, N]), alpha, epi, _lib.current_stream()), "gemm")
    ref = alpha * (a.double() @ w.double().T)
    if epi & 1:
        ref = ref + bias.double()
    if epi & 2:
        ref = torch.relu(ref)
    if epi & 4:
        ref = torch.nn.functional.gelu(ref)
    if epi & 8:
        ref = ref + res.double()
    assert rel_err(ref.cpu().numpy(), out.cpu().numpy()) < FP32_REL_TOL


@pytest.mark.parametrize("M, N, K, epi", [(1100, 3076, 96, 5),     # 2 x 9 x 65 = 1170 tiles of 128 x 48: several rounds of three per CU, ragged in M and N
                                          (1024, 3072, 64, 9),     # 1024 tiles: whole rounds of two per CU, the deep-ring kernel
                                          (3000, 2308, 160, 1)])   # 2 x 24 x 49 = 2352 tiles
def test_k_contiguous_gemm_several_rounds_of_workgroups(tuning, M, N, K, epi):
    """The library's own choice between the deep-ring and the lean 128 x 48 kernel on problems of several rounds of
    workgroups, against the same product with 64 x 48 tiles forced and against float64."""
    lib = _lib.library()
    rng = np.random.default_rng(M + N + K)
    a = torch.from_numpy(rng.normal(size=(2, M, K)).astype(np.float32)).cuda()
    w = torch.from_numpy(rng.normal(size=(N, K)).astype(np.float32)).cuda()
    bias = torch.from_numpy(rng.normal(size=N).astype(np.float32)).cuda()
    res = torch.from_numpy(rng.normal(size=(2, M, N)).astype(np.float32)).cuda()

    def product():
        out = torch.full((2, M, N), float("nan"), device="cuda")
        _lib.check(lib.mi355x_gemm_f32(a.data_ptr(), w.data_ptr(), out.data_ptr(), bias.data_ptr(), res.data_ptr(), 1, 2, M, N, K,
                                       _lib.i64_array([0, M * K, K, 1]), _lib.i64_array([0, 0, 1, K]), _lib.i64_array([0, M * N, N]),
                                       _lib.i64_array([0, M * N, N]), 1.0, epi, _lib.current_stream()), "gemm")
        return out

    tuning()
    chosen = product()
    tuning(MI355X_GEMM_NT_BN=48, MI355X_GEMM_NT_PER_CU=2)
    small_tiles = product()
    ref = a.double() @ w.double().T + bias.double()
    if epi & 4:
        ref = torch.nn.functional.gelu(ref)
    if epi & 8:
        ref = ref + res.double()
    assert rel_err(ref.cpu().numpy(), chosen.cpu().numpy()) < FP32_REL_TOL
    # the same products in another order of summation (one chain against two k-split chains): fp32 rounding apart
    torch.testing.assert_close(chosen, small_tiles, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("variables", [{"MI355X_GEMM_CONFIG": c} for c in range(5)] + [{"MI355X_GEMM_NT_BK": 32},
                                                                                        {"MI355X_GEMM_NT_BK": 32, "MI355X_GEMM_NT_BN": 64},
                                                                                        {"MI355X_GEMM_GROUP_M": 1}, {"MI355X_GEMM_KSPLIT": 1},
                                       {"MI355X_GEMM_NT_BM": 128, "MI355X_GEMM_NT_BN": 48, "MI355X_GEMM_NT_BK": 32}])
@pytest.mark.parametrize("M, N, K, epi", [(130, 100, 64, 9), (257, 52, 2112, 5)])
def test_forced_gemm_variants(tuning, variables, M, N, K, epi):
    """Every tile shape of the generic double-buffered kernel (which the library itself only picks for operands that are
    not both k-contiguous), the 32-k walk of the k-contiguous kernel where it would pick 64-k tiles, and a forced
    panel height, on the k-contiguous problem: each must give the float64 product within the fp32 bar."""
    tuning(**variables)
    lib = _lib.library()
    rng = np.random.default_rng(M + N + K)
    a = torch.from_numpy(rng.normal(size=(M, K)).astype(np.float32)).cuda()
    w = torch.from_numpy(rng.normal(size=(N, K)).astype(np.float32)).cuda()
    bias = torch.from_numpy(rng.normal(size=N).astype(np.float32)).cuda()
    res = torch.from_numpy(rng.normal(size=(M, N)).astype(np.float32)).cuda()
    out = torch.full((M, N), float("nan"), device="cuda")
    _lib.check(lib.mi355x_gemm_f32(a.data_ptr(), w.data_ptr(), out.data_ptr(), bias.data_ptr(), res.data_ptr(), 1, 1, M, N, K,
                                   _lib.i64_array([0, 0, K, 1]), _lib.i64_array([0, 0, 1, K]), _lib.i64_array([0, 0, N]),
                                   _lib.i64_array([0, 0, N]), 1.0, epi, _lib.current_stream()), "gemm")
    ref = a.double() @ w.double().T + bias.double()
    if epi & 4:
        ref = torch.nn.functional.gelu(ref)
    if epi & 8:
        ref = ref + res.double()
    assert rel_err(ref.cpu().numpy(), out.cpu().numpy()) < FP32_REL_TOL


@pytest.mark.parametrize("config", range(5))
def test_forced_conv_tile_variants(tuning, config):
    """MI355X_CONV_CONFIG sends a convolution the gather kernel would take to each tile shape of the generic kernel."""
    tuning(MI355X_CONV_CONFIG=config)
    rng = np.random.default_rng(40 + config)
    x = rng.normal(size=(2, 32, 13, 11)).astype(np.float32)
    w = (rng.normal(size=(40, 32, 3, 3)) / 17.0).astype(np.float32)
    b = rng.normal(size=40).astype(np.float32)
    y = np.zeros((2, 40, 13, 11), np.float32)
    donnx.ONNXConv(X=x, W=w, B=b, Y=y, pads=[1, 1, 1, 1])
    assert rel_err(O.conv2d(x, w, b, pads=(1, 1, 1, 1)), y) < FP32_REL_TOL


@pytest.mark.parametrize("variables", [{"MI355X_MMI_GENERIC": 1}, {"MI355X_MMI_WGS_PER_CU": 1}, {"MI355X_MMI_WGS_PER_CU": 2},
                                       {"MI355X_MMI_TILE": 128}, {"MI355X_MMI_TILE": 256}, {"MI355X_MMI_TILE": 129},
                                       {"MI355X_MMI_TILE": 257}])
@pytest.mark.parametrize("M, N, K", [(384, 272, 192), (300, 208, 64), (1000, 400, 320)])
def test_forced_matmul_integer_variants(tuning, variables, M, N, K):
    """Every form of MatMulInteger on shapes the library would give to another one: the generic kernel, the persistent
    kernel with fewer workgroups per CU, one 128 x 128 or 256 x 192 tile per workgroup, and the two measurement variants
    that read A straight from global memory. Signed and unsigned operands, one zero point per operand and one per row /
    column; bit-exact against the int64 formula."""
    tuning(**variables)
    lib = _lib.library()
    rng = np.random.default_rng(55 + M)
    for a_unsigned, b_unsigned, per_axis in ((0, 0, False), (0, 0, True), (1, 0, False), (0, 1, True), (1, 1, False)):
        A = rng.integers(0, 256, size=(M, K)).astype(np.uint8) if a_unsigned else rng.integers(-128, 128, size=(M, K)).astype(np.int8)
        B = rng.integers(0, 256, size=(K, N)).astype(np.uint8) if b_unsigned else rng.integers(-128, 128, size=(K, N)).astype(np.int8)
        za = rng.integers(0, 100, size=M if per_axis else 1).astype(A.dtype)
        zb = rng.integers(0, 100, size=N if per_axis else 1).astype(B.dtype)
        ta, tb, tza, tzb = (torch.from_numpy(v).cuda() for v in (A, B, za, zb))
        y = torch.full((M, N), -7, dtype=torch.int32, device="cuda")
        _lib.check(lib.mi355x_matmul_integer(ta.data_ptr(), tb.data_ptr(), tza.data_ptr(), tzb.data_ptr(), y.data_ptr(), M, N, K,
                                             a_unsigned, b_unsigned, za.size, zb.size, _lib.current_stream()), "matmul_integer")
        want = (A.astype(np.int64) - za.astype(np.int64).reshape(-1, 1)) @ (B.astype(np.int64) - zb.astype(np.int64).reshape(1, -1))
        assert np.array_equal(want.astype(np.int32), y.cpu().numpy()), (variables, a_unsigned, b_unsigned, per_axis)


def test_matmul_integer_long_k_takes_the_wide_tile_and_matches(c_oracle):
    """K >= 1536 on a shape whose 256 x 192 tiles fill the CUs: the library picks the one-tile-per-workgroup kernel by
    itself; checked against the C restatement on every element and against the checksum identity."""
    rng = np.random.default_rng(56)
    A = rng.integers(-128, 128, size=(2048, 1536), dtype=np.int8)
    B = rng.integers(-128, 128, size=(1536, 1536), dtype=np.int8)
    Y = np.zeros((2048, 1536), np.int32)
    donnx.ONNXMatMulInteger(A=A, B=B, a_zero_point=np.array(-5, np.int8), b_zero_point=np.array(7, np.int8), Y=Y)
    assert np.array_equal(c_oracle.matmul_integer(A, B, -5, 7), Y)
    ca = A.astype(np.int64).sum(0) + 5 * 2048
    rb = B.astype(np.int64).sum(1) - 7 * 1536
    assert int(Y.astype(np.int64).sum()) == int(ca @ rb)


def test_save_transients_keeps_every_intermediate(golden):
    # the reference's ONNXModel(save_transients=...) (tests/test_bert_subgraphs.py:37-52): intermediates are
    # kept, so the graph runs node by node; each saved tensor is checked against the oracle's value
    hidden, heads, ffn, bsz, seq = (int(v) for v in golden["bert_meta"])
    w = {k[len("bert_"):]: golden[k] for k in golden.files if k.startswith("bert_") and k not in
         ("bert_x", "bert_y", "bert_meta")}
    saved = {}
    model = donnx.ONNXModel("bert_saved", bert_encoder_layer_model(w, bsz, seq, heads), save_transients=saved)
    got = model(golden["bert_x"])
    assert rel_err(golden["bert_y"], got) < FP32_REL_TOL
    assert model.compile_and_init().num_launches == 26        # nothing was fused away
    x = golden["bert_x"]
    d = hidden // heads
    q = O.add(O.matmul(x, w["wq"]), w["bq"])
    q_heads = O.transpose(O.reshape(q, (bsz, seq, heads, d)), (0, 2, 1, 3))
    k_heads = O.transpose(O.reshape(O.add(O.matmul(x, w["wk"]), w["bk"]), (bsz, seq, heads, d)), (0, 2, 1, 3))
    probs = O.softmax(O.matmul(q_heads, O.transpose(k_heads, (0, 1, 3, 2))) / np.float32(np.sqrt(d)), axis=3)
    for name, expected in (("q_lin", q), ("q_heads", q_heads), ("probs", probs)):
        assert rel_err(expected, saved[name].cpu().numpy()) < FP32_REL_TOL, name
    assert {"attn_res", "h1", "inter", "ffn_res", "ctx"} <= set(saved) and "y" not in saved
    with pytest.raises(ValueError, match="not with use_hip_graph"):
        donnx.ONNXModel("bert_saved_graph", bert_encoder_layer_model(w, bsz, seq, heads), save_transients={},
                        use_hip_graph=True)


@pytest.mark.parametrize("seq", [40, 200, 384])
def test_bert_layer_other_sequence_lengths(seq):
    # sequence lengths other than the benchmark's 128: the fused attention kernel walks the keys in blocks
    rng = np.random.default_rng(seq)
    w = O.bert_layer_weights(rng, hidden=256, ffn=512)
    for k in ("bq", "bk", "bv", "bo", "b1", "b2"):
        w[k] = rng.normal(0.0, 0.02, size=w[k].shape).astype(np.float32)
    x = rng.normal(size=(3, seq, 256)).astype(np.float32)
    model = donnx.ONNXModel(f"bert_seq{seq}", bert_encoder_layer_model(w, 3, seq, 4))
    got = model(x)
    assert model.compile_and_init().num_launches == 7
    assert rel_err(O.bert_layer(x, w, heads=4), got) < FP32_REL_TOL


@pytest.mark.parametrize("c_shape", [(12, ), (6, 12)])
@pytest.mark.parametrize("act", ["Relu", "Gelu"])
def test_gemm_addend_then_activation(c_shape, act):
    # act(A B + C): a row bias folds with the activation into one launch; a full [M, N] addend must be added
    # before the activation, so the activation stays its own launch (the epilogue adds a residual last)
    H, T = proto.helper, proto.TensorProto
    rng = np.random.default_rng(len(c_shape))
    a, b, c = (rng.normal(size=s).astype(np.float32) for s in ((6, 8), (8, 12), c_shape))
    nodes = [H.make_node("Gemm", ["a", "b", "c"], ["g"]), H.make_node(act, ["g"], ["y"])]
    g = H.make_graph(nodes, "g", [H.make_tensor_value_info("a", T.FLOAT, [6, 8]), H.make_tensor_value_info("b", T.FLOAT, [8, 12]),
                                  H.make_tensor_value_info("c", T.FLOAT, list(c_shape))],
                     [H.make_tensor_value_info("y", T.FLOAT, [6, 12])])
    model = donnx.ONNXModel(f"gemm_{act}_{len(c_shape)}", H.make_model(g, opset_imports=[H.make_opsetid("", 12)]))
    got = model(a, b, c)
    pre = O.gemm(a, b, c)
    assert rel_err(O.relu(pre) if act == "Relu" else O.gelu(pre), got) < FP32_REL_TOL
    assert model.compile_and_init().num_launches == (1 if len(c_shape) == 1 else 2)


def test_pad_then_conv_matches_padding_by_hand():
    # Pad(constant 0, spatial) -> Conv(pads) -> Relu as one convolution launch, against the oracle's convolution
    # of the explicitly padded input
    from test_fusion import _pad_conv_model
    m = _pad_conv_model([0, 0, 1, 2, 0, 0, 3, 0], conv_pads=[1, 0, 0, 2])
    x = np.random.default_rng(6).normal(size=(2, 3, 8, 8)).astype(np.float32)
    w = [t for t in m.graph.initializer if t.name == "w"][0].array.reshape(4, 3, 3, 3)
    model = donnx.ONNXModel("pad_conv_values", m)
    got = model(x)
    xp = np.pad(x, ((0, 0), (0, 0), (1, 3), (2, 0)))
    assert rel_err(O.conv2d(xp, w, None, pads=(1, 0, 0, 2)), got) < FP32_REL_TOL
    assert model.compile_and_init().num_launches == 1


@pytest.mark.parametrize("fuse", [True, False])
def test_tanh_gelu_silu_softplus_chain_values(fuse):
    from test_fusion import _chain_model, _tanh_gelu_and_silu_nodes
    nodes, consts = _tanh_gelu_and_silu_nodes()
    x = np.random.default_rng(8).normal(scale=2, size=(4, 8)).astype(np.float32)
    got = donnx.ONNXModel(f"tanh_chain_{fuse}", _chain_model(nodes, consts), fuse=fuse)(x)
    x64 = x.astype(np.float64)
    gelu = 0.5 * x64 * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x64 + 0.044715 * x64 ** 3)))
    silu = gelu / (1.0 + np.exp(-gelu))
    assert np.allclose(got, np.log1p(np.exp(silu)), rtol=1e-5, atol=1e-6)


def test_classifier_head_with_log_softmax_reductions_and_sum():
    """Gemm -> LogSoftmax, plus ReduceSum / ReduceMax / ReduceMin of the logits and a three-input Sum, in one
    ONNXModel: the operators of pure_implementations.py:301-343, 529-616 on the importer's path."""
    H, T = proto.helper, proto.TensorProto
    rng = np.random.default_rng(9)
    x = rng.normal(size=(16, 64)).astype(np.float32)
    w = rng.normal(scale=0.2, size=(10, 64)).astype(np.float32)
    b = rng.normal(scale=0.1, size=(10, )).astype(np.float32)
    nodes = [H.make_node("Gemm", ["x", "w", "b"], ["logits"], transB=1),
             H.make_node("LogSoftmax", ["logits"], ["logp"], axis=1),
             H.make_node("ReduceSum", ["logits"], ["rs"], axes=[1], keepdims=1),
             H.make_node("ReduceMax", ["logits"], ["rmax"], axes=[1], keepdims=1),
             H.make_node("ReduceMin", ["logits"], ["rmin"], axes=[0], keepdims=0),
             H.make_node("Sum", ["logp", "logits", "logp"], ["total"])]
    outs = [("logp", [16, 10]), ("rs", [16, 1]), ("rmax", [16, 1]), ("rmin", [10]), ("total", [16, 10])]
    g = H.make_graph(nodes, "head", [H.make_tensor_value_info("x", T.FLOAT, [16, 64])],
                     [H.make_tensor_value_info(n, T.FLOAT, s) for n, s in outs],
                     initializer=[proto.numpy_helper.from_array(w, "w"), proto.numpy_helper.from_array(b, "b")])
    model = donnx.ONNXModel("classifier_head", H.make_model(g, opset_imports=[H.make_opsetid("", 12)]))
    logp, rs, rmax, rmin, total = model(x)
    logits = O.gemm(x, w, b, transB=1)
    assert rel_err(O.log_softmax(logits, axis=1), logp) < FP32_REL_TOL
    assert rel_err(O.reduce_sum(logits, [1]), rs) < FP32_REL_TOL
    assert np.allclose(rmax, O.reduce_max(logits, [1]), rtol=1e-5) and np.allclose(rmin, O.reduce_min(logits, [0], 0), rtol=1e-5)
    assert rel_err(O.sum_(O.log_softmax(logits, axis=1), logits, O.log_softmax(logits, axis=1)), total) < FP32_REL_TOL


# ----------------------------------------------------------------------------- the reference's ONNX file fixtures
def test_reference_slice_fixture():
    # tests/test_bert_subgraphs.py:17-26 of the reference, on its own data file
    model = donnx.ONNXModel("slice_fixture", proto.load(os.path.join(GOLDEN_DIR, "slice.onnx")), fold_constants=False)
    out = model(data=torch.ones(2, device="cuda"))
    assert out.shape == (1, ) and out[0] == 1.0
    out = model(data=torch.tensor([3.0, 7.0], device="cuda"))
    assert out.tolist() == [3.0]


@pytest.mark.parametrize("fold", [False, True])
def test_reference_bert_subgraph_fixture(fold):
    """tests/test_bert_subgraphs.py:29-52 and tests/transformation/test_constant_folding.py:17-41 of the
    reference, on its own data file: a model without inputs (Slice of the position embeddings, Cast of the
    target shape, Reshape); same result with and without constant folding; the saved Cast result equals the
    shape weight."""
    m = proto.load(os.path.join(GOLDEN_DIR, "reshape.onnx"))
    weights = {t.name: np.asarray(t.array).reshape(t.dims) for t in m.graph.initializer}
    saved = {}
    model = donnx.ONNXModel(f"bert_subgraph_{fold}", m, fold_constants=fold, save_transients=None if fold else saved)
    out = model()
    emb = weights["bert/embeddings/position_embeddings:0"]
    expected = O.slice_(emb, weights["const_slice__40"], weights["const_slice__41"]).reshape(1, 256, 768)
    assert tuple(out.shape) == (1, 256, 768) and np.array_equal(np.asarray(out), expected)   # no inputs: numpy result
    if not fold:
        cast = saved["bertSLASHembeddingsSLASHReshape_4__42COLON0"]
        assert cast.dtype == torch.int64
        assert torch.equal(cast.type(torch.int32).cpu(), model.weights["bert/embeddings/Reshape_4/shape:0"].cpu())


@pytest.mark.parametrize("conv_bias", [True, False])
@pytest.mark.parametrize("fuse", [True, False])
def test_conv_batchnorm_relu_values(conv_bias, fuse):
    # Conv -> BatchNormalization -> Relu: folded into one convolution launch, or three launches, against the
    # oracle's convolution followed by the inference batch normalization
    from test_fusion import _conv_bn_model
    m, w, p = _conv_bn_model(conv_bias=conv_bias)
    x = np.random.default_rng(11).normal(size=(2, 3, 8, 8)).astype(np.float32)
    model = donnx.ONNXModel(f"conv_bn_values_{conv_bias}_{fuse}", m, fuse=fuse)
    got = model(x)
    conv = O.conv2d(x, w, p["cb"] if conv_bias else None, pads=(1, 1, 1, 1))
    expected = O.relu(O.batch_normalization(conv, p["scale"], p["beta"], p["mean"], p["var"], 1e-3))
    assert rel_err(expected, got) < FP32_REL_TOL
    assert model.compile_and_init().num_launches == (1 if fuse else 3)


@pytest.mark.parametrize("shape, wshape, pads, strides", [
    ((4, 64, 28, 28), (64, 64, 3, 3), [1, 1, 1, 1], [1, 1]),      # K % 32 == 0: the gather kernel, 16-byte stores
    ((2, 32, 15, 15), (48, 32, 3, 3), [1, 1, 1, 1], [2, 2]),      # 8 x 8 output
    ((3, 3, 9, 11), (5, 3, 3, 3), [0, 1, 2, 0], [1, 1]),          # generic kernel, OH * OW odd: scalar stores
    ((2, 16, 8, 8), (16, 16, 1, 1), [0, 0, 0, 0], [1, 1])])       # 1 x 1 projection shortcut
@pytest.mark.parametrize("epi", [_lib.EPI_RESIDUAL, _lib.EPI_BIAS | _lib.EPI_RESIDUAL | _lib.EPI_RELU_AFTER,
                                 _lib.EPI_BIAS | _lib.EPI_RELU | _lib.EPI_RESIDUAL | _lib.EPI_RELU_AFTER])
def test_conv_residual_epilogue(shape, wshape, pads, strides, epi):
    """relu?(relu?(conv + bias) + residual) in the convolution's epilogue against the oracle's Conv, Add, Relu."""
    rng = np.random.default_rng(12)
    x = rng.normal(size=shape).astype(np.float32)
    w = (rng.normal(size=wshape) / np.sqrt(np.prod(wshape[1:]))).astype(np.float32)
    b = rng.normal(size=wshape[0]).astype(np.float32)
    pre = O.conv2d(x, w, b if epi & _lib.EPI_BIAS else None, strides=tuple(strides), pads=tuple(pads))
    r = rng.normal(size=pre.shape).astype(np.float32)
    expected = (O.relu(pre) if epi & _lib.EPI_RELU else pre) + r
    expected = O.relu(expected) if epi & _lib.EPI_RELU_AFTER else expected
    tx, tw, tb, tr = (torch.from_numpy(a).cuda() for a in (x, w, b, r))
    y = torch.full(pre.shape, float("nan"), device="cuda")
    lib = _lib.library()
    args = [tx.data_ptr(), tw.data_ptr(), tb.data_ptr() if epi & _lib.EPI_BIAS else None, tr.data_ptr(), y.data_ptr(),
            *shape, wshape[0], wshape[2], wshape[3], _lib.i64_array(pads), _lib.i64_array(strides), _lib.i64_array([1, 1]),
            epi, torch.cuda.current_stream().cuda_stream]
    assert lib.mi355x_conv2d_res_f32(*args) == 0, lib.mi355x_last_error()
    torch.cuda.synchronize()
    assert rel_err(expected, y.cpu().numpy()) < FP32_REL_TOL
    # the flags are checked: a residual flag without a residual, or an unknown flag, launches nothing
    args[3] = None
    assert lib.mi355x_conv2d_res_f32(*args) == 1 and b"without residual" in lib.mi355x_last_error()
    assert lib.mi355x_conv2d_f32(*(args[:3] + args[4:-2] + [_lib.EPI_RESIDUAL, None])) == 1


@pytest.mark.parametrize("shape, wshape, tail", [
    ((3, 32, 20, 20), (64, 32, 3, 3), 2),      # 1200 positions: 18.75 tiles of 64 -> 16 whole tiles, 44 slices, the last one ragged
    ((2, 64, 16, 16), (80, 64, 3, 3), 7),      # two tiles of output channels (the second partly filled), 1 whole tile per row of tiles
    ((1, 32, 9, 9), (16, 32, 3, 3), 1)])       # 81 positions, odd: scalar stores in the slices
@pytest.mark.parametrize("epi", [0, _lib.EPI_BIAS | _lib.EPI_RELU, _lib.EPI_BIAS | _lib.EPI_RESIDUAL | _lib.EPI_RELU_AFTER])
@pytest.mark.parametrize("per_cu", [None, 2])   # the lean kernel the library takes (three workgroups per CU), the six-deep ring
def test_conv_last_round_as_slices(tuning, shape, wshape, tail, epi, per_cu):
    """The convolution's last round of tiles run as 16-position slices (the library chooses that by the number of
    tiles and CUs; here it is forced on small problems through MI355X_CONV_TAIL = number of position tiles to slice)."""
    rng = np.random.default_rng(31 + tail)
    x = rng.normal(size=shape).astype(np.float32)
    w = (rng.normal(size=wshape) / np.sqrt(np.prod(wshape[1:]))).astype(np.float32)
    b = rng.normal(size=wshape[0]).astype(np.float32)
    pre = O.conv2d(x, w, b if epi & _lib.EPI_BIAS else None, strides=(1, 1), pads=(1, 1, 1, 1))
    r = rng.normal(size=pre.shape).astype(np.float32)
    expected = O.relu(pre) if epi & _lib.EPI_RELU else pre
    expected = expected + r if epi & _lib.EPI_RESIDUAL else expected
    expected = O.relu(expected) if epi & _lib.EPI_RELU_AFTER else expected
    tx, tw, tb, tr = (torch.from_numpy(a).cuda() for a in (x, w, b, r))
    lib = _lib.library()
    args = lambda y: [tx.data_ptr(), tw.data_ptr(), tb.data_ptr() if epi & _lib.EPI_BIAS else None,
                      tr.data_ptr() if epi & _lib.EPI_RESIDUAL else None, y.data_ptr(), *shape, wshape[0], 3, 3,
                      _lib.i64_array([1, 1, 1, 1]), _lib.i64_array([1, 1]), _lib.i64_array([1, 1]), epi,
                      torch.cuda.current_stream().cuda_stream]
    results = []
    for setting in (str(tail), "0"):
        tuning(MI355X_CONV_TAIL=setting, MI355X_CONV_PER_CU=per_cu)
        y = torch.full(pre.shape, float("nan"), device="cuda")
        assert lib.mi355x_conv2d_res_f32(*args(y)) == 0, lib.mi355x_last_error()
        torch.cuda.synchronize()
        results.append(y.cpu().numpy())
    assert rel_err(expected, results[0]) < FP32_REL_TOL
    # a slice adds up the same products in the same order as the tile it stands in for
    assert np.array_equal(results[0], results[1])


@pytest.mark.parametrize("shape, wshape, strides, pads, dilations, gather_bn", [
    ((2, 32, 12, 12), (64, 32, 3, 3), (1, 1), (1, 1, 1, 1), (1, 1), 64),     # one window of 9 steps
    ((1, 64, 14, 14), (48, 64, 3, 3), (1, 1), (1, 1, 1, 1), (1, 1), 128),    # the unrolled 18 steps once, wide tiles
    ((2, 96, 11, 13), (64, 96, 3, 3), (2, 2), (1, 0, 2, 1), (1, 1), 64),     # 27 steps: 18 + a remainder of 9; stride 2, uneven pads
    ((1, 160, 9, 9), (32, 160, 3, 3), (1, 1), (2, 2, 2, 2), (2, 2), 128),    # 45 steps, dilation 2
    ((1, 32, 10, 7), (16, 32, 1, 9), (1, 1), (0, 4, 0, 4), (1, 1), 64),      # nine taps in one row
    ((3, 64, 9, 9), (64, 64, 1, 1), (1, 1), (0, 0, 0, 0), (1, 1), 64),       # 1 x 1
    ((2, 224, 8, 8), (40, 224, 1, 1), (2, 2), (0, 0, 0, 0), (1, 1), 128)])   # 1 x 1, stride 2, 7 steps
def test_conv_taps_known_at_compile_time(tuning, shape, wshape, strides, pads, dilations, gather_bn):
    """3 x 3 and 1 x 1 filters over a multiple of 32 channels take a gather whose tap offsets are compile-time
    register choices plus a scalar channel offset; MI355X_CONV_STATIC_TAPS=0 sends the same call through the tap
    table, MI355X_CONV_PER_CU=2 through the six-deep register ring instead of the lean kernel (64-position tiles
    only). All add up the same products in the same order."""
    rng = np.random.default_rng(77 + shape[1])
    x = rng.normal(size=shape).astype(np.float32)
    w = (rng.normal(size=wshape) / np.sqrt(np.prod(wshape[1:]))).astype(np.float32)
    b = rng.normal(size=wshape[0]).astype(np.float32)
    expected = O.relu(O.conv2d(x, w, b, strides=strides, pads=pads, dilations=dilations))
    tx, tw, tb = (torch.from_numpy(a).cuda() for a in (x, w, b))
    lib = _lib.library()
    results = []
    for setting, per_cu in (("1", None), ("0", None), ("1", 2), ("0", 2)):
        tuning(MI355X_CONV_GATHER_BN=gather_bn, MI355X_CONV_STATIC_TAPS=setting, MI355X_CONV_PER_CU=per_cu)
        y = torch.full(expected.shape, float("nan"), device="cuda")
        status = lib.mi355x_conv2d_f32(tx.data_ptr(), tw.data_ptr(), tb.data_ptr(), y.data_ptr(), *shape, wshape[0], wshape[2], wshape[3],
                                       _lib.i64_array(pads), _lib.i64_array(strides), _lib.i64_array(dilations),
                                       _lib.EPI_BIAS | _lib.EPI_RELU, torch.cuda.current_stream().cuda_stream)
        assert status == 0, lib.mi355x_last_error()
        torch.cuda.synchronize()
        results.append(y.cpu().numpy())
    assert rel_err(expected, results[0]) < FP32_REL_TOL
    for other in results[1:]:
        assert np.array_equal(results[0], other)


def test_tasklet_fusion_programs_values():
    # tests/transformation/test_tasklet_fusion.py:9-60 of the reference: same inputs (ones, twos), same expectations
    from test_fusion import _tasklet_fusion_graphs
    A, B = np.ones((5, 5), np.float32), np.ones((5, 5), np.float32) * 2
    for name, (m, inputs, fn) in _tasklet_fusion_graphs().items():
        result = donnx.ONNXModel("tf_values_" + name, m)(*([A, B][:len(inputs)]))
        assert np.allclose(result, fn(A, B)), name


def test_outputs_that_are_inputs_or_weights():
    # a graph output may be a graph input or an initializer itself: each comes back as a copy in a buffer of its own
    H, T = proto.helper, proto.TensorProto
    g = H.make_graph([H.make_node("Relu", ["x"], ["r"])], "g", [H.make_tensor_value_info("x", T.FLOAT, [2, 3])],
                     [H.make_tensor_value_info("x", T.FLOAT, [2, 3]), H.make_tensor_value_info("r", T.FLOAT, [2, 3]),
                      H.make_tensor_value_info("w", T.FLOAT, [3])],
                     initializer=[proto.numpy_helper.from_array(np.arange(3, dtype=np.float32), "w")])
    model = donnx.ONNXModel("passthrough", H.make_model(g, opset_imports=[H.make_opsetid("", 12)]))
    x = np.random.default_rng(13).normal(size=(2, 3)).astype(np.float32)
    same, relu, w = model(x)
    assert np.array_equal(same, x) and np.array_equal(relu, np.maximum(x, 0)) and np.array_equal(w, np.arange(3, dtype=np.float32))
    xt = torch.from_numpy(x).cuda()
    same_t, _, _ = model(xt)
    assert same_t.data_ptr() != xt.data_ptr() and torch.equal(same_t, xt)
    # the model with no node at all
    g0 = H.make_graph([], "g0", [H.make_tensor_value_info("x", T.FLOAT, [2, 3])], [H.make_tensor_value_info("x", T.FLOAT, [2, 3])])
    assert np.array_equal(donnx.ONNXModel("empty", H.make_model(g0, opset_imports=[H.make_opsetid("", 12)]))(x), x)


def test_view_into_a_callers_buffer_that_is_read_earlier():
    """A transient whose reshaped view is a caller-owned array is normally produced straight into that array. Not when
    something reads the array before the view is taken: state 1 computes t = -x and y1 = relu(buf), state 2 makes buf the
    reshaped t. y1 must see what the caller passed in buf, and buf must hold -x afterwards."""
    from dace_onnx_amd.util import utils
    sdfg = dace.SDFG("read_then_view")
    for name, shape in (("x", [2, 3]), ("buf", [3, 2]), ("y1", [3, 2])):
        sdfg.add_array(name, shape, dace.float32)
    sdfg.add_transient("t", [2, 3], dace.float32)
    s1 = sdfg.add_state("compute")
    neg, relu = donnx.ONNXNeg("neg"), donnx.ONNXRelu("relu")
    for node, src, dst in ((neg, "x", "t"), (relu, "buf", "y1")):
        node.add_in_connector("X")
        node.add_out_connector("Y")
        s1.add_edge(s1.add_read(src), None, node, "X", sdfg.make_array_memlet(src))
        s1.add_edge(node, "Y", s1.add_write(dst), None, sdfg.make_array_memlet(dst))
    s2 = sdfg.add_state("view")
    alias = dace.AliasNode("reshape", "data", "reshaped")
    s2.add_edge(s2.add_read("t"), None, alias, "data", sdfg.make_array_memlet("t"))
    s2.add_edge(alias, "reshaped", s2.add_write("buf"), None, sdfg.make_array_memlet("buf"))
    utils.expand_onnx_nodes(sdfg)
    compiled = dace.CompiledSDFG(sdfg)
    assert [item[0] for item in compiled._plan] == ["call", "call", "alias"]
    rng = np.random.default_rng(21)
    x = torch.from_numpy(rng.normal(size=(2, 3)).astype(np.float32)).cuda()
    buf = torch.from_numpy(rng.normal(size=(3, 2)).astype(np.float32)).cuda()
    before = buf.clone()
    y1 = torch.full((3, 2), float("nan"), device="cuda")
    compiled(x=x, buf=buf, y1=y1)
    torch.cuda.synchronize()
    assert torch.equal(y1, torch.relu(before))
    assert torch.equal(buf, (-x).reshape(3, 2))


def test_conv_network_hip_graph_replays_match_eager():
    """A convolution network (Conv+BatchNormalization+Relu folded, MaxPool through LDS, residual epilogue, global
    average pooling, Gemm, LogSoftmax) replayed as one HIP graph: every replay, with eager work and synchronisation
    in between and changing inputs, equals the eager result bit for bit."""
    H, T = proto.helper, proto.TensorProto
    rng = np.random.default_rng(14)
    f32 = lambda *s: rng.normal(size=s).astype(np.float32)
    inits = {"w1": f32(16, 3, 3, 3) * 0.2, "b1": f32(16), "s1": f32(16), "be1": f32(16), "m1": f32(16),
             "v1": rng.uniform(0.5, 2.0, size=16).astype(np.float32), "w2": f32(16, 16, 3, 3) * 0.1, "wf": f32(10, 16), "bf": f32(10)}
    nodes = [H.make_node("Conv", ["x", "w1", "b1"], ["c1"], pads=[1, 1, 1, 1]),
             H.make_node("BatchNormalization", ["c1", "s1", "be1", "m1", "v1"], ["n1"]), H.make_node("Relu", ["n1"], ["r1"]),
             H.make_node("MaxPool", ["r1"], ["p1"], kernel_shape=[3, 3], strides=[2, 2], pads=[1, 1, 1, 1]),
             H.make_node("Conv", ["p1", "w2"], ["c2"], pads=[1, 1, 1, 1]), H.make_node("Add", ["c2", "p1"], ["a2"]),
             H.make_node("Relu", ["a2"], ["r2"]), H.make_node("GlobalAveragePool", ["r2"], ["g"]),
             H.make_node("Flatten", ["g"], ["f"], axis=1), H.make_node("Gemm", ["f", "wf", "bf"], ["l"], transB=1),
             H.make_node("LogSoftmax", ["l"], ["y"], axis=1)]
    g = H.make_graph(nodes, "cnn", [H.make_tensor_value_info("x", T.FLOAT, [8, 3, 64, 64])],
                     [H.make_tensor_value_info("y", T.FLOAT, [8, 10])],
                     initializer=[proto.numpy_helper.from_array(v, k) for k, v in inits.items()])
    m = H.make_model(g, opset_imports=[H.make_opsetid("", 12)])
    model = donnx.ONNXModel("cnn_graph", m, use_hip_graph=True)
    assert model.compile_and_init().num_launches == 6     # conv, maxpool, conv + residual + relu, mean, gemm, logsoftmax
    xs = [torch.from_numpy(f32(8, 3, 64, 64)).cuda() for _ in range(3)]
    model(xs[0])                                          # first call runs eagerly and captures
    for i in range(5):
        xi = xs[i % 3]
        replayed = model(xi).clone()
        torch.cuda.synchronize()
        ref = donnx.ONNXModel(f"cnn_eager_{i}", m)(xi)
        assert torch.equal(replayed, ref), i
    # and the values: against the oracle, node by node
    x = xs[1].cpu().numpy()
    r1 = O.relu(O.batch_normalization(O.conv2d(x, inits["w1"], inits["b1"], pads=(1, 1, 1, 1)), inits["s1"], inits["be1"], inits["m1"], inits["v1"]))
    p1 = O.maxpool2d(r1, (3, 3), (2, 2), (1, 1, 1, 1))
    r2 = O.relu(O.conv2d(p1, inits["w2"], None, pads=(1, 1, 1, 1)) + p1)
    logits = O.gemm(O.global_average_pool(r2).reshape(8, 16), inits["wf"], inits["bf"], transB=1)
    assert rel_err(O.log_softmax(logits, axis=1), model(xs[1]).cpu().numpy()) < FP32_REL_TOL

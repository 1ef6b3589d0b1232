"""Seeded random shapes, layouts and attributes through the C ABI, against float64 references.

The fixed cases elsewhere pin the benchmark configurations and the edge cases the reference tests; these
sweep what lies between them -- ragged and aligned extents, either operand contiguous along k or not,
broadcast batches, every epilogue combination, pads / strides / dilations, zero points present or absent --
so that each kernel variant and each of their tile choices is reached with extents that do not divide its
tiles. Every case is printed (and flushed) before it is launched."""
import numpy as np
import pytest
import torch

from dace_onnx_amd import _lib
from conftest import FP32_REL_TOL

pytestmark = pytest.mark.gpu


def _lib_and_stream():
    return _lib.library(), _lib.current_stream


def _rel(got, ref):
    return ((got.double() - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item() if ref.numel() else 0.0


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_gemm(seed):
    lib, stream = _lib_and_stream()
    rng, dev, failures = np.random.default_rng(seed), "cuda", []
    for case in range(60):
        b0, b1 = int(rng.choice([1, 1, 2, 3])), int(rng.choice([1, 1, 2, 5]))
        if rng.random() < 0.6:
            M = int(rng.choice([1, 16, 63, 64, 100, 128, 257, 512]))
            N, K = 4 * int(rng.integers(1, 80)), 32 * int(rng.integers(1, 12))
        else:
            M, N, K = (int(v) for v in rng.integers(1, 150, size=3))
        a_kc, b_kc = rng.random() < 0.7, rng.random() < 0.6       # contiguous along k?
        a_bcast, b_bcast = rng.random() < 0.15, rng.random() < 0.3

        def operand(rows, cols, rows_major, bcast):
            shape = (1 if bcast else b0, 1 if bcast else b1) + ((rows, cols) if rows_major else (cols, rows))
            t = torch.from_numpy(rng.normal(size=shape).astype(np.float32)).to(dev)
            return t, (t if rows_major else t.transpose(2, 3)).expand(b0, b1, rows, cols)

        _, A = operand(M, K, a_kc, a_bcast)
        _, B = operand(K, N, not b_kc, b_bcast)
        epi = int(rng.choice([0, 1, 2, 3, 4, 5, 8, 9, 13]))
        alpha = float(rng.choice([1.0, 0.5, -2.0]))
        bias = torch.from_numpy(rng.normal(size=N).astype(np.float32)).to(dev)
        res = torch.from_numpy(rng.normal(size=(b0, b1, M, N)).astype(np.float32)).to(dev)
        C = torch.full((b0, b1, M, N), float("nan"), device=dev)
        ref = alpha * (A.double() @ B.double())
        if epi & _lib.EPI_BIAS:
            ref = ref + bias.double()
        if epi & _lib.EPI_RELU:
            ref = torch.relu(ref)
        if epi & _lib.EPI_GELU:
            ref = torch.nn.functional.gelu(ref)
        if epi & _lib.EPI_RESIDUAL:
            ref = ref + res.double()
        tag = f"gemm seed {seed} case {case}: b{b0}x{b1} M{M} N{N} K{K} a_kc={a_kc} b_kc={b_kc} " \
              f"bcast={a_bcast},{b_bcast} epi={epi} alpha={alpha}"
        print(tag, flush=True)
        s4 = lambda v: _lib.i64_array([v.stride(i) for i in range(4)])
        s3 = lambda v: _lib.i64_array([v.stride(i) for i in range(3)])
        st = lib.mi355x_gemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), bias.data_ptr(), res.data_ptr(), b0, b1, M, N,
                                 K, s4(A), s4(B), s3(C), s3(res), alpha, epi, stream())
        torch.cuda.synchronize()
        if st != 0 or torch.isnan(C).any().item() or _rel(C, ref) >= FP32_REL_TOL:
            failures.append(tag)
    assert not failures, failures


def test_random_gemm_many_tiles():
    """Both operands k-contiguous, outputs of several hundred to several thousand tiles: the shapes on which the
    library chooses between 64 x 48 and 128 x 48 tiles, between the deep and the lean register ring and between one,
    two and three workgroups per CU, with extents that leave partial tiles and partial rounds of workgroups."""
    lib, stream = _lib_and_stream()
    rng, dev, failures = np.random.default_rng(7), "cuda", []
    for case in range(24):
        b1 = int(rng.choice([1, 1, 1, 2]))
        M, N, K = int(rng.integers(500, 4600)), 4 * int(rng.integers(150, 1100)), 32 * int(rng.integers(1, 24))
        if case % 6 == 0:   # whole rounds of two workgroups per CU: the pattern that keeps the deep ring
            M, N, b1 = 128 * int(rng.choice([8, 16, 32])), 48 * 64, 1
        A = torch.from_numpy(rng.normal(size=(1, b1, M, K)).astype(np.float32)).to(dev)
        W = torch.from_numpy(rng.normal(size=(N, K)).astype(np.float32)).to(dev)
        epi = int(rng.choice([0, 1, 5, 9]))
        bias = torch.from_numpy(rng.normal(size=N).astype(np.float32)).to(dev)
        res = torch.from_numpy(rng.normal(size=(1, b1, M, N)).astype(np.float32)).to(dev)
        C = torch.full((1, b1, M, N), float("nan"), device=dev)
        ref = A.double() @ W.double().T
        if epi & _lib.EPI_BIAS:
            ref = ref + bias.double()
        if epi & _lib.EPI_GELU:
            ref = torch.nn.functional.gelu(ref)
        if epi & _lib.EPI_RESIDUAL:
            ref = ref + res.double()
        tag = f"gemm many tiles case {case}: b{b1} M{M} N{N} K{K} epi={epi}"
        print(tag, flush=True)
        st = lib.mi355x_gemm_f32(A.data_ptr(), W.data_ptr(), C.data_ptr(), bias.data_ptr(), res.data_ptr(), 1, b1, M, N, K,
                                 _lib.i64_array([0, M * K, K, 1]), _lib.i64_array([0, 0, 1, K]), _lib.i64_array([0, M * N, N]),
                                 _lib.i64_array([0, M * N, N]), 1.0, epi, stream())
        torch.cuda.synchronize()
        if st != 0 or torch.isnan(C).any().item() or _rel(C, ref) >= FP32_REL_TOL:
            failures.append(tag)
        del A, W, C, ref, res
    assert not failures, failures


@pytest.mark.parametrize("seed", [0, 1])
def test_random_conv(seed):
    lib, stream = _lib_and_stream()
    rng, failures = np.random.default_rng(100 + seed), []
    for case in range(60):
        kh, kw = int(rng.choice([1, 2, 3, 5])), int(rng.choice([1, 2, 3, 5]))
        if rng.random() < 0.7:   # C KH KW a multiple of 32: the gather kernel
            c = int(rng.choice([32, 64, 96, 128, 192]))
        else:
            c = int(rng.integers(1, 40))
        n, m = int(rng.integers(1, 5)), int(rng.choice([1, 7, 16, 48, 64, 65, 100, 130, 200]))
        h, w = int(rng.integers(kh, 30)), int(rng.integers(kw, 30))
        sh, sw, dh, dw = (int(v) for v in rng.integers(1, 3, size=4))
        pt, pl, pb, pr = (int(v) for v in rng.integers(0, 3, size=4))
        if h + pt + pb < (kh - 1) * dh + 1 or w + pl + pr < (kw - 1) * dw + 1:
            continue
        epi = int(rng.choice([0, 1, 2, 3]))
        x = torch.from_numpy(rng.normal(size=(n, c, h, w)).astype(np.float32))
        wt = torch.from_numpy(rng.normal(size=(m, c, kh, kw)).astype(np.float32))
        b = torch.from_numpy(rng.normal(size=m).astype(np.float32))
        ref = torch.nn.functional.conv2d(torch.nn.functional.pad(x.double(), (pl, pr, pt, pb)), wt.double(),
                                         b.double() if epi & 1 else None, stride=(sh, sw), dilation=(dh, dw))
        if epi & 2:
            ref = torch.relu(ref)
        y = torch.full(ref.shape, float("nan"), device="cuda")
        xd, wd, bd = x.cuda(), wt.cuda(), b.cuda()
        tag = f"conv seed {seed} case {case}: N{n} C{c} H{h} W{w} M{m} k{kh}x{kw} pads {pt},{pl},{pb},{pr} " \
              f"s{sh},{sw} d{dh},{dw} epi{epi}"
        print(tag, flush=True)
        st = lib.mi355x_conv2d_f32(xd.data_ptr(), wd.data_ptr(), bd.data_ptr(), y.data_ptr(), n, c, h, w, m, kh, kw,
                                   _lib.i64_array([pt, pl, pb, pr]), _lib.i64_array([sh, sw]), _lib.i64_array([dh, dw]),
                                   epi, stream())
        torch.cuda.synchronize()
        if st != 0 or torch.isnan(y).any().item() or _rel(y.cpu(), ref) >= FP32_REL_TOL:
            failures.append(tag)
    assert not failures, failures


def test_random_matmul_integer():
    lib, stream = _lib_and_stream()
    rng, dev, failures = np.random.default_rng(200), "cuda", []
    for case in range(60):
        if rng.random() < 0.6:    # the persistent kernel: K a multiple of 128, N of 4
            M, N, K = int(rng.choice([1, 31, 128, 129, 300, 640])), 4 * int(rng.integers(1, 120)), 128 * int(rng.integers(1, 8))
        else:
            M, N, K = (int(v) for v in rng.integers(1, 300, size=3))
        A = torch.randint(-128, 128, (M, K), dtype=torch.int8, device=dev)
        B = torch.randint(-128, 128, (K, N), dtype=torch.int8, device=dev)
        za, zb = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
        use_a, use_b = (bool(v) for v in rng.random(2) < 0.7)
        zat, zbt = torch.tensor([za], dtype=torch.int8, device=dev), torch.tensor([zb], dtype=torch.int8, device=dev)
        Y = torch.full((M, N), -7, dtype=torch.int32, device=dev)
        tag = f"mmi case {case}: {M}x{N}x{K} za={za if use_a else None} zb={zb if use_b else None}"
        print(tag, flush=True)
        st = lib.mi355x_matmul_integer_i8(A.data_ptr(), B.data_ptr(), zat.data_ptr() if use_a else None,
                                          zbt.data_ptr() if use_b else None, Y.data_ptr(), M, N, K, stream())
        torch.cuda.synchronize()
        ref = (A.cpu().long() - (za if use_a else 0)) @ (B.cpu().long() - (zb if use_b else 0))
        if st != 0 or not torch.equal(Y.cpu().long(), ref):     # bit-exact
            failures.append(tag)
    assert not failures, failures


def test_random_rowwise_kernels():
    lib, stream = _lib_and_stream()
    rng, dev, failures = np.random.default_rng(300), "cuda", []
    for case in range(40):
        outer, n = int(rng.integers(1, 300)), int(rng.choice([1, 3, 64, 128, 129, 500, 1024, 4100]))
        inner = int(rng.choice([1, 1, 1, 2, 7]))
        tag = f"softmax / reduce_mean case {case}: {outer}x{n}x{inner}"
        print(tag, flush=True)
        X = torch.from_numpy(rng.normal(size=(outer, n, inner)).astype(np.float32)).to(dev) * 3
        Y = torch.empty_like(X)
        st = lib.mi355x_softmax_f32(X.data_ptr(), Y.data_ptr(), outer, n, inner, stream())
        torch.cuda.synchronize()
        if st != 0 or (Y.double() - torch.softmax(X.double(), 1)).abs().max().item() >= 1e-6:
            failures.append("softmax " + tag)
        Ym = torch.empty(outer, inner, device=dev)
        st = lib.mi355x_reduce_mean_f32(X.data_ptr(), Ym.data_ptr(), outer, n, inner, stream())
        torch.cuda.synchronize()
        if st != 0 or (Ym.double() - X.double().mean(1)).abs().max().item() >= 1e-5:
            failures.append("reduce_mean " + tag)
    for case in range(40):
        rows, cols = int(rng.integers(1, 500)), int(rng.choice([1, 4, 64, 100, 768, 769, 1024, 3000, 5000]))
        has_bias = bool(rng.random() < 0.7)
        tag = f"layernorm case {case}: {rows}x{cols} bias={has_bias}"
        print(tag, flush=True)
        X = torch.from_numpy(rng.normal(size=(rows, cols)).astype(np.float32)).to(dev) * 2 + 1
        g = torch.from_numpy(rng.normal(size=cols).astype(np.float32)).to(dev)
        b = torch.from_numpy(rng.normal(size=cols).astype(np.float32)).to(dev)
        Y = torch.empty_like(X)
        st = lib.mi355x_layernorm_f32(X.data_ptr(), g.data_ptr(), b.data_ptr() if has_bias else None, Y.data_ptr(), rows,
                                      cols, 1e-5, stream())
        torch.cuda.synchronize()
        ref = torch.nn.functional.layer_norm(X.double(), (cols, ), g.double(), b.double() if has_bias else None, 1e-5)
        if st != 0 or _rel(Y, ref) >= FP32_REL_TOL:
            failures.append(tag)
    assert not failures, failures


def test_random_attention():
    lib, stream = _lib_and_stream()
    rng, dev, failures = np.random.default_rng(400), "cuda", []
    for case in range(30):
        b0, b1, sq = int(rng.integers(1, 4)), int(rng.integers(1, 6)), int(rng.choice([1, 16, 50, 64, 65, 128, 200]))
        scale = float(rng.choice([0.125, 1.0, 0.3]))
        sk = int(rng.choice([128, 128, 1, 77, 130, 300, 512]))
        tag = f"attention case {case}: b{b0}x{b1} sq{sq} sk{sk} scale{scale}"
        print(tag, flush=True)
        # Q, K, V as slices of one packed projection result, heads interleaved: the strided form the fusion produces
        pack = torch.from_numpy(rng.normal(size=(b0, max(sq, sk), b1, 3, 64)).astype(np.float32)).to(dev)
        q, k, v = pack[:, :sq, :, 0], pack[:, :sk, :, 1], pack[:, :sk, :, 2]
        out = torch.full((b0, sq, b1, 64), float("nan"), device=dev)
        st3 = lambda t: _lib.i64_array([t.stride(0), t.stride(2), t.stride(1)])
        st = lib.mi355x_attention_f32(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), b0, b1, sq, sk, 64,
                                      st3(q), st3(k), st3(v), st3(out), scale, stream())
        torch.cuda.synchronize()
        Q, K, V = (t.permute(0, 2, 1, 3).double() for t in (q, k, v))
        ref = torch.softmax(scale * (Q @ K.transpose(-1, -2)), -1) @ V
        if st != 0 or torch.isnan(out).any().item() or _rel(out.permute(0, 2, 1, 3), ref) >= FP32_REL_TOL:
            failures.append(tag)
    assert not failures, failures

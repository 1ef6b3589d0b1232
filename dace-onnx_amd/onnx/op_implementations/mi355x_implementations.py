"""The ``"mi355x"`` expansions: ONNX library nodes -> calls into libmi355x_onnx.so.

Each class has the shape of a reference expansion (``ONNXForward`` with
``forward_can_be_applied`` / ``forward``, registered through
``op_implementation(op=..., name="mi355x")``) and stands where the reference has
its ``"pure"`` / ``"cuDNN"`` classes:

==================  ============================================================
MatMul              PureMatMul -> PureEinsum, pure_implementations.py:130-267
Gemm                PureGemm, pure_implementations.py:433-459
Conv                PureConv2D, img_op_implementations.py:164-326;
                    CudnnConvolution, cudnn_implementations.py:111-336
MatMulInteger       (ONNX Runtime only, onnx_op.py:686-687)
Softmax             PureSoftmax, pure_implementations.py:346-366
LayerNormalization  (exporter decomposition, pure_implementations.py:97-109 etc.)
Add/Sub/Mul/Div     python_pure_op_implementation, pure_implementations.py:77-94
Relu, Erf, Sqrt     pure_implementations.py:462-474, 112-127, 41-56
Pow                 PurePow, pure_implementations.py:59-74
Log, Reciprocal,    PureLog :23-38, PureReciprocal :275-293, Tanh :296-298,
Tanh, Softplus,     Softplus :696-698, PureSigmoid :701-712
Sigmoid
Exp, Neg, Abs       (ONNX Runtime only in the reference)
Gelu                (exporter decomposition Div, Erf, Add, Mul, Mul)
ReduceMean/Sum/     PureReduceMean :97-109, PureReduceSum / Max / Min :301-343
Max/Min
LogSoftmax          PureLogSoftmax, pure_implementations.py:594-616
Sum                 PureSum, pure_implementations.py:529-591
Einsum              PureEinsum, pure_implementations.py:238-267
Cast                PureCast, pure_implementations.py:382-430
Slice               PureSlice, pure_implementations.py:619-693
Transpose           PureTranspose, pure_implementations.py:369-379
Reshape, Flatten    PureReshape / PureFlatten, pure_implementations.py:477-526
Identity            pure_implementations.py:270-272
==================  ============================================================

``forward_can_be_applied`` mirrors every precondition of the kernel it would
call, so an unsupported configuration is refused before anything is launched
(and, there being no ONNX Runtime here, reported as an error by the fallback).
``forward`` returns a :class:`~dace_onnx_amd.sdfg.KernelCall`.
"""
import numpy as np

from ... import sdfg as dace
from ... import _lib
from ...sdfg import SDFG, SDFGState, Ptr, Stream, I64Array, U32Array, F32Array, PtrArray, AliasNode
from ...util.utils import in_desc_with_name, out_desc_with_name, prod
from ..forward_implementation_abc import ONNXForward
from .utils import op_implementation, kernel_call_for_node

IMPLEMENTATION_NAME = "mi355x"
MAX_ELTWISE_DIMS = 8


def _is_f32(*descs) -> bool:
    return all(d.dtype == dace.float32 for d in descs)


def _contig(*descs) -> bool:
    return all(d.is_contiguous() for d in descs)


def _has_input(node, state, name) -> bool:
    return any(e.dst_conn == name for e in state.in_edges(node))


def _has_output(node, state, name) -> bool:
    return any(e.src_conn == name for e in state.out_edges(node))


def _broadcast_shape(*shapes):
    try:
        return tuple(np.broadcast_shapes(*shapes))
    except ValueError:
        return None


def _broadcast_strides(desc, out_shape):
    """Element strides of ``desc`` in the index space of ``out_shape`` (0 where broadcast)."""
    pad = len(out_shape) - len(desc.shape)
    strides = []
    for d, extent in enumerate(out_shape):
        if d < pad or desc.shape[d - pad] == 1:
            strides.append(0)
        else:
            strides.append(desc.strides[d - pad])
    return strides


# ------------------------------------------------------------------------------------
# contractions


class _BatchPlan:
    """How a numpy-style batched matmul maps onto the kernel's two batch levels."""

    def __init__(self, A, B, Y):
        self.ok = False
        if len(A.shape) < 2 or len(B.shape) < 2:
            return
        M, K = A.shape[-2:]
        K2, N = B.shape[-2:]
        if K != K2:
            return
        batch = _broadcast_shape(A.shape[:-2], B.shape[:-2])
        if batch is None or tuple(Y.shape) != tuple(batch) + (M, N) or Y.strides[-1] != 1 and N != 1:
            return
        a_bs = _broadcast_strides(dace.Array(A.dtype, A.shape[:-2], A.strides[:-2]), batch)
        b_bs = _broadcast_strides(dace.Array(B.dtype, B.shape[:-2], B.strides[:-2]), batch)
        y_bs = list(Y.strides[:-2])
        dims = [(e, a, b, y) for e, a, b, y in zip(batch, a_bs, b_bs, y_bs) if e != 1]
        a_sm, a_sk = A.strides[-2:]
        b_sk, b_sn = B.strides[-2:]
        y_sm = Y.strides[-2]
        # B shared by every batch entry: fold batch dims into M while A and Y allow it
        while dims and dims[-1][2] == 0 and dims[-1][1] == M * a_sm and dims[-1][3] == M * y_sm:
            M *= dims[-1][0]
            dims.pop()
        # merge adjacent batch dims that all three operands walk as one
        merged = []
        for d in dims:
            if merged:
                e0, a0, b0, y0 = merged[-1]
                if a0 == d[1] * d[0] and b0 == d[2] * d[0] and y0 == d[3] * d[0]:
                    merged[-1] = (e0 * d[0], d[1], d[2], d[3])
                    continue
            merged.append(d)
        if len(merged) > 2:
            return
        while len(merged) < 2:
            merged.insert(0, (1, 0, 0, 0))
        (self.batch0, a0, b0, y0), (self.batch1, a1, b1, y1) = merged
        self.M, self.N, self.K = M, N, K
        self.a_strides = [a0, a1, a_sm, a_sk]
        self.b_strides = [b0, b1, b_sk, b_sn]
        self.c_strides = [y0, y1, y_sm]
        self.ok = True


def _gemm_call(node, state, plan, a_conn, b_conn, y_conn, bias_conn=None, residual_conn=None,
               r_strides=None, alpha=1.0, epilogue=_lib.EPI_NONE, offsets=(0, 0, 0)):
    return kernel_call_for_node(node, state, "mi355x_gemm_f32", [
        Ptr(a_conn, offsets[0]), Ptr(b_conn, offsets[1]), Ptr(y_conn, offsets[2]), Ptr(bias_conn), Ptr(residual_conn),
        plan.batch0, plan.batch1, plan.M, plan.N, plan.K,
        I64Array(plan.a_strides), I64Array(plan.b_strides), I64Array(plan.c_strides),
        I64Array(r_strides) if r_strides is not None else None,
        float(alpha), int(epilogue), Stream()])


def _fused_epilogue(node, state, sdfg, plan):
    """Epilogue requested by the fusion pass through private node attributes
    (the reference passes per-node tuning the same way: ``node._algorithm``,
    cudnn_implementations.py:251-254). Extra inputs use the connectors
    ``_bias`` ([N]) and ``_residual`` (same shape as Y)."""
    epi = 0
    bias_conn = residual_conn = r_strides = None
    if _has_input(node, state, "_bias"):
        epi |= _lib.EPI_BIAS
        bias_conn = "_bias"
    act = getattr(node, "_activation", None)
    if act == "relu":
        epi |= _lib.EPI_RELU
    elif act == "gelu":
        epi |= _lib.EPI_GELU
    if _has_input(node, state, "_residual"):
        epi |= _lib.EPI_RESIDUAL
        residual_conn = "_residual"
        r = in_desc_with_name(node, state, sdfg, "_residual")
        y = out_desc_with_name(node, state, sdfg, "Y")
        if tuple(r.shape) != tuple(y.shape) or tuple(r.strides) != tuple(y.strides):
            raise ValueError("fused residual must have the shape and layout of Y")
        r_strides = plan.c_strides
    return epi, bias_conn, residual_conn, r_strides


@op_implementation(op="MatMul", name=IMPLEMENTATION_NAME)
class MI355XMatMul(ONNXForward):
    """numpy-style (batched, broadcasting) matmul on the fp32 MFMA GEMM kernel.
    Leading dimensions become the kernel's batch levels, or part of M when B is
    shared; nothing is copied or transposed."""

    @staticmethod
    def _operands(node, state, sdfg):
        """Descriptors of A, B, Y as the kernel will address them: the arrays on the
        edges, or the (shape, strides[, element offset]) views the fusion pass attached."""
        descs = []
        for conn, attr, getter in (("A", "_a_view", in_desc_with_name), ("B", "_b_view", in_desc_with_name),
                                   ("Y", "_y_view", out_desc_with_name)):
            d = getter(node, state, sdfg, conn)
            view = getattr(node, attr, None)
            descs.append(dace.Array(d.dtype, view[0], view[1]) if view else d)
        return descs

    @staticmethod
    def _offsets(node):
        """Element offsets of the A, B, Y views into the arrays on the edges."""
        views = [getattr(node, attr, None) for attr in ("_a_view", "_b_view", "_y_view")]
        return tuple(int(v[2]) if v and len(v) > 2 else 0 for v in views)

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        A, B, Y = MI355XMatMul._operands(node, state, sdfg)
        if len(A.shape) == 1 or len(B.shape) == 1:  # same refusal as PureMatMul (:133-140)
            return False
        if not _is_f32(A, B, Y):
            return False
        return _BatchPlan(A, B, Y).ok

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        A, B, Y = MI355XMatMul._operands(node, state, sdfg)
        plan = _BatchPlan(A, B, Y)
        if not plan.ok:
            raise ValueError(f"{node.label}: operand layout cannot be expressed as a strided batched GEMM")
        epi, bias_conn, residual_conn, r_strides = _fused_epilogue(node, state, sdfg, plan)
        return _gemm_call(node, state, plan, "A", "B", "Y", bias_conn, residual_conn, r_strides,
                          alpha=getattr(node, "_alpha", 1.0), epilogue=epi, offsets=MI355XMatMul._offsets(node))


def _einsum_plan(equation, X0, X1, Y):
    """A two-operand einsum as one strided batched GEMM: (plan, swapped) or None.

    Letters are sorted into batch (in both inputs and the output), M (first input and output), N (second
    input and output) and K (both inputs, not the output). All K letters must be walked as one axis by both
    inputs; the last M and the last N letter are the GEMM's m and n, every other output letter is a batch
    axis in which the operand that does not carry it is broadcast (stride 0) -- ``_BatchPlan`` folds such
    axes back into M where the layout allows. The output's innermost letter must be an N letter (n stride 1);
    when it is an M letter the two inputs change roles. Not expressible this way (and refused): ellipses,
    a letter repeated inside one term, a letter that only one input carries and the output does not."""
    eq = equation.replace(" ", "")
    if "..." in eq or "->" not in eq:
        return None
    lhs, out = eq.split("->")
    terms = lhs.split(",")
    if len(terms) != 2 or any(not t.isalpha() for t in terms) or (out and not out.isalpha()):
        return None
    t0, t1 = terms
    descs = {0: X0, 1: X1}
    if len(t0) != len(X0.shape) or len(t1) != len(X1.shape) or len(out) != len(Y.shape):
        return None
    if len(set(t0)) != len(t0) or len(set(t1)) != len(t1) or len(set(out)) != len(out):
        return None
    size = {}
    for term, d in ((t0, X0), (t1, X1), (out, Y)):
        for letter, extent in zip(term, d.shape):
            if size.setdefault(letter, extent) != extent:
                return None
    if not set(out) <= set(t0) | set(t1) or (set(t0) ^ set(t1)) - set(out):
        return None
    swapped = bool(out) and out[-1] in t0 and out[-1] not in t1      # innermost output letter must come from "B"
    if swapped:
        t0, t1 = t1, t0
        descs = {0: X1, 1: X0}
    stride = lambda term, d, letter: d.strides[term.index(letter)] if letter in term else 0
    m_letters = [c for c in out if c in t0 and c not in t1]
    n_letters = [c for c in out if c in t1 and c not in t0]
    k_letters = [c for c in t0 if c in t1 and c not in out]
    batch = [c for c in out if c not in m_letters[-1:] and c not in n_letters[-1:]]
    # K letters as one axis of both inputs
    K, a_sk, b_sk = 1, 0, 0
    for c in reversed(k_letters):
        sa, sb = stride(t0, descs[0], c), stride(t1, descs[1], c)
        if K == 1:
            a_sk, b_sk = sa, sb
        elif sa != a_sk * K or sb != b_sk * K:
            return None
        K *= size[c]
    m, n = (m_letters[-1:] or [None])[0], (n_letters[-1:] or [None])[0]
    M, N = (size[m] if m else 1), (size[n] if n else 1)
    shape_b = [size[c] for c in batch]
    view = lambda term, d, tail_shape, tail: dace.Array(Y.dtype, shape_b + tail_shape,
                                                         [stride(term, d, c) for c in batch] + tail)
    A = view(t0, descs[0], [M, K], [stride(t0, descs[0], m) if m else 0, a_sk])
    B = view(t1, descs[1], [K, N], [b_sk, stride(t1, descs[1], n) if n else 0])
    C = view(out, Y, [M, N], [stride(out, Y, m) if m else 0, stride(out, Y, n) if n else 1])
    plan = _BatchPlan(A, B, C)
    return (plan, swapped) if plan.ok else None


@op_implementation(op="Einsum", name=IMPLEMENTATION_NAME)
class MI355XEinsum(ONNXForward):
    """Two-operand fp32 contractions on the MFMA GEMM kernel, nothing copied or transposed (the reference
    lowers Einsum -- and through it every MatMul -- to DaCe's einsum SDFG: PureEinsum, :238-267)."""

    @staticmethod
    def _plan(node, state, sdfg):
        conns = sorted((c for c in node.in_connectors if c.startswith("Inputs__")), key=lambda c: int(c[len("Inputs__"):]))
        if len(conns) != 2 or not node.equation:
            return None
        X0, X1 = (in_desc_with_name(node, state, sdfg, c) for c in conns)
        Y = out_desc_with_name(node, state, sdfg, "Output")
        if not _is_f32(X0, X1, Y) or not _contig(Y):
            return None
        equation = node.equation.decode() if isinstance(node.equation, bytes) else node.equation
        found = _einsum_plan(equation, X0, X1, Y)
        return None if found is None else (found[0], conns[::-1] if found[1] else conns)

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        return MI355XEinsum._plan(node, state, sdfg) is not None

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        plan, (a_conn, b_conn) = MI355XEinsum._plan(node, state, sdfg)
        return _gemm_call(node, state, plan, a_conn, b_conn, "Output")


@op_implementation(op="Gemm", name=IMPLEMENTATION_NAME)
class MI355XGemm(ONNXForward):
    """``Y = alpha * A' B' + beta * C``. transA / transB are strides; ``C`` is
    fused as a row bias (shape [N] or [1,N]) or as a full [M,N] addend.
    PureGemm only accepts alpha=1, beta=1, transA=0, transB=1 (:436-440)."""

    @staticmethod
    def _c_kind(C, M, N):
        if C is None:
            return "none"
        shape = tuple(C.shape)
        if shape in ((N, ), (1, N)) and C.strides[-1] == 1:
            return "bias"
        if shape == (M, N) and C.strides[-1] == 1:
            return "full"
        return None

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        A = in_desc_with_name(node, state, sdfg, "A")
        B = in_desc_with_name(node, state, sdfg, "B")
        Y = out_desc_with_name(node, state, sdfg, "Y")
        C = in_desc_with_name(node, state, sdfg, "C") if _has_input(node, state, "C") else None
        if len(A.shape) != 2 or len(B.shape) != 2 or len(Y.shape) != 2:
            return False
        if not _is_f32(A, B, Y) or (C is not None and not _is_f32(C)):
            return False
        M, K = (A.shape[1], A.shape[0]) if node.transA else A.shape
        K2, N = (B.shape[1], B.shape[0]) if node.transB else B.shape
        if K != K2 or tuple(Y.shape) != (M, N) or Y.strides[-1] != 1:
            return False
        if C is not None and node.beta not in (0.0, 1.0):
            return False
        if C is not None and node.beta == 1.0 and MI355XGemm._c_kind(C, M, N) is None:
            return False
        return True

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        A = in_desc_with_name(node, state, sdfg, "A")
        B = in_desc_with_name(node, state, sdfg, "B")
        Y = out_desc_with_name(node, state, sdfg, "Y")
        C = in_desc_with_name(node, state, sdfg, "C") if _has_input(node, state, "C") else None
        if node.transA:
            A = dace.Array(A.dtype, A.shape[::-1], A.strides[::-1])
        if node.transB:
            B = dace.Array(B.dtype, B.shape[::-1], B.strides[::-1])
        plan = _BatchPlan(A, B, Y)
        assert plan.ok
        kind = MI355XGemm._c_kind(C, plan.M, plan.N) if (C is not None and node.beta == 1.0) else "none"
        epi, bias_conn, residual_conn, r_strides = 0, None, None, None
        if kind == "bias":
            epi, bias_conn = _lib.EPI_BIAS, "C"
        elif kind == "full":
            epi, residual_conn, r_strides = _lib.EPI_RESIDUAL, "C", [0, 0, C.strides[0]]
        act = getattr(node, "_activation", None)
        if act == "relu":
            epi |= _lib.EPI_RELU
        elif act == "gelu":
            epi |= _lib.EPI_GELU
        return _gemm_call(node, state, plan, "A", "B", "Y", bias_conn, residual_conn, r_strides,
                          alpha=float(node.alpha), epilogue=epi)


def _conv_geometry(node, X, W):
    """(pads[4], strides[2], dilations[2], out_h, out_w) under ONNX rules, or None."""
    if len(X.shape) != 4 or len(W.shape) != 4:
        return None
    H, Wd = X.shape[2:]
    KH, KW = W.shape[2:]
    strides = list(node.strides) if node.strides is not None else [1, 1]
    dil = list(node.dilations) if node.dilations is not None else [1, 1]
    if len(strides) != 2 or len(dil) != 2 or min(strides + dil) < 1:
        return None
    if node.kernel_shape is not None and list(node.kernel_shape) != [KH, KW]:
        return None
    eff = [(KH - 1) * dil[0] + 1, (KW - 1) * dil[1] + 1]
    auto_pad = node.auto_pad or "NOTSET"
    if auto_pad == "NOTSET":
        pads = list(node.pads) if node.pads is not None else [0, 0, 0, 0]
        if len(pads) != 4 or min(pads) < 0:
            return None
    elif auto_pad == "VALID":
        pads = [0, 0, 0, 0]
    elif auto_pad in ("SAME_UPPER", "SAME_LOWER"):
        pads = [0, 0, 0, 0]
        for i, (size, s) in enumerate(((H, strides[0]), (Wd, strides[1]))):
            out = -(-size // s)
            total = max((out - 1) * s + eff[i] - size, 0)
            lo = total // 2 if auto_pad == "SAME_UPPER" else total - total // 2
            pads[i], pads[i + 2] = lo, total - lo
    else:
        return None
    hin, win = H + pads[0] + pads[2], Wd + pads[1] + pads[3]
    if hin < eff[0] or win < eff[1]:
        return None
    return pads, strides, dil, (hin - eff[0]) // strides[0] + 1, (win - eff[1]) // strides[1] + 1


@op_implementation(op="Conv", name=IMPLEMENTATION_NAME)
class MI355XConv(ONNXForward):
    """2-D NCHW convolution as implicit GEMM on MFMA. Honours ``strides``,
    ``pads`` (also asymmetric), ``dilations`` and ``auto_pad``; the bias, a
    following Relu, a residual Add and the Relu after it (attached by the fusion pass as ``_activation``,
    ``_residual``, ``_activation_after``) are applied in the kernel's epilogue. PureConv2D refuses any
    non-zero pad and ignores the stride (img_op_implementations.py:201-203,278)."""

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        X = in_desc_with_name(node, state, sdfg, "X")
        W = in_desc_with_name(node, state, sdfg, "W")
        Y = out_desc_with_name(node, state, sdfg, "Y")
        B = in_desc_with_name(node, state, sdfg, "B") if _has_input(node, state, "B") else None
        if not _is_f32(X, W, Y) or not _contig(X, W, Y):
            return False
        if len(X.shape) != 4 or len(W.shape) != 4:  # only 2-D, like the pure and cuDNN versions
            return False
        if node.group != 1 or X.shape[1] != W.shape[1]:
            return False
        geom = _conv_geometry(node, X, W)
        if geom is None:
            return False
        if tuple(Y.shape) != (X.shape[0], W.shape[0], geom[3], geom[4]):
            return False
        if B is not None and (not _is_f32(B) or tuple(B.shape) != (W.shape[0], ) or not _contig(B)):
            return False
        if prod(X.shape) >= 2**30 or prod(Y.shape) >= 2**31:
            return False
        if _has_input(node, state, "_residual"):     # attached by the fusion pass: a tensor exactly like Y
            R = in_desc_with_name(node, state, sdfg, "_residual")
            if not _is_f32(R) or not _contig(R) or tuple(R.shape) != tuple(Y.shape):
                return False
        elif getattr(node, "_activation_after", None):
            return False
        return getattr(node, "_activation", None) in (None, "relu") and getattr(node, "_activation_after", None) in (None, "relu")

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        X = in_desc_with_name(node, state, sdfg, "X")
        W = in_desc_with_name(node, state, sdfg, "W")
        has_bias, has_res = _has_input(node, state, "B"), _has_input(node, state, "_residual")
        pads, strides, dil, _, _ = _conv_geometry(node, X, W)
        epi = (_lib.EPI_BIAS if has_bias else 0) | (_lib.EPI_RELU if getattr(node, "_activation", None) == "relu" else 0)
        N, C, H, Wd = X.shape
        M, _, KH, KW = W.shape
        geometry = [N, C, H, Wd, M, KH, KW, I64Array(pads), I64Array(strides), I64Array(dil)]
        if not has_res:
            return kernel_call_for_node(node, state, "mi355x_conv2d_f32", [
                Ptr("X"), Ptr("W"), Ptr("B" if has_bias else None), Ptr("Y")] + geometry + [epi, Stream()])
        epi |= _lib.EPI_RESIDUAL | (_lib.EPI_RELU_AFTER if getattr(node, "_activation_after", None) == "relu" else 0)
        return kernel_call_for_node(node, state, "mi355x_conv2d_res_f32", [
            Ptr("X"), Ptr("W"), Ptr("B" if has_bias else None), Ptr("_residual"), Ptr("Y")] + geometry + [epi, Stream()])


@op_implementation(op="MaxPool", name=IMPLEMENTATION_NAME)
class MI355XMaxPool(ONNXForward):
    """2-D max pooling with pads, strides and dilations (floor output size, no ``Indices`` output).
    PureMaxPool2D (img_op_implementations.py:28-161) refuses pads and dilations."""

    @staticmethod
    def _geometry(node, X):
        if node.kernel_shape is None or len(node.kernel_shape) != 2 or len(X.shape) != 4:
            return None
        window = dace.Array(X.dtype, [1, 1] + [int(k) for k in node.kernel_shape])
        geom = _conv_geometry(node, X, window)
        if geom is None:
            return None
        pads, strides, dil, oh, ow = geom
        eff = [(window.shape[2] - 1) * dil[0] + 1, (window.shape[3] - 1) * dil[1] + 1]
        if max(pads[0], pads[2]) >= eff[0] or max(pads[1], pads[3]) >= eff[1]:
            return None                 # a window entirely inside the padding has no maximum
        return pads, strides, dil, oh, ow

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        X = in_desc_with_name(node, state, sdfg, "X")
        Y = out_desc_with_name(node, state, sdfg, "Y")
        if _has_output(node, state, "Indices") or (node.ceil_mode or 0) != 0 or (node.storage_order or 0) != 0:
            return False
        if not _is_f32(X, Y) or not _contig(X, Y):
            return False
        geom = MI355XMaxPool._geometry(node, X)
        return geom is not None and tuple(Y.shape) == (X.shape[0], X.shape[1], geom[3], geom[4])

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        X = in_desc_with_name(node, state, sdfg, "X")
        pads, strides, dil, _, _ = MI355XMaxPool._geometry(node, X)
        return kernel_call_for_node(node, state, "mi355x_maxpool2d_f32", [
            Ptr("X"), Ptr("Y"), X.shape[0], X.shape[1], X.shape[2], X.shape[3], int(node.kernel_shape[0]),
            int(node.kernel_shape[1]), I64Array(pads), I64Array(strides), I64Array(dil), Stream()])


@op_implementation(op="GlobalAveragePool", name=IMPLEMENTATION_NAME)
class MI355XGlobalAveragePool(ONNXForward):
    """Mean over the spatial axes (GlobalAveragePool, img_op_implementations.py:410-412): the row mean of
    ``[N * C, H * W]``."""

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        X = in_desc_with_name(node, state, sdfg, "X")
        Y = out_desc_with_name(node, state, sdfg, "Y")
        return _is_f32(X, Y) and _contig(X, Y) and len(X.shape) >= 3 and prod(X.shape[2:]) >= 1 and \
            tuple(Y.shape) == tuple(X.shape[:2]) + (1, ) * (len(X.shape) - 2)

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        X = in_desc_with_name(node, state, sdfg, "X")
        return kernel_call_for_node(node, state, "mi355x_reduce_mean_f32",
                                    [Ptr("X"), Ptr("Y"), prod(X.shape[:2]), prod(X.shape[2:]), 1, Stream()])


@op_implementation(op="BatchNormalization", name=IMPLEMENTATION_NAME)
class MI355XBatchNormalization(ONNXForward):
    """Inference form: the stored mean and variance are used, only ``Y`` is produced. (The reference's
    PureBatchNormalization, img_op_implementations.py:329-407, is the training form -- batch statistics and
    running-mean update -- and is not provided here; a node with the training outputs is refused.)"""

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        if any(_has_output(node, state, c) for c in ("out_mean", "out_var", "saved_mean", "saved_var")):
            return False
        X = in_desc_with_name(node, state, sdfg, "X")
        Y = out_desc_with_name(node, state, sdfg, "Y")
        if not _is_f32(X, Y) or not _contig(X, Y) or len(X.shape) < 2 or tuple(X.shape) != tuple(Y.shape):
            return False
        for conn in ("scale", "B", "in_mean", "in_var"):
            if not _has_input(node, state, conn):
                return False
            d = in_desc_with_name(node, state, sdfg, conn)
            if not _is_f32(d) or not _contig(d) or tuple(d.shape) != (X.shape[1], ):
                return False
        return True

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        X = in_desc_with_name(node, state, sdfg, "X")
        eps = 1e-5 if node.epsilon is None else float(node.epsilon)
        return kernel_call_for_node(node, state, "mi355x_batchnorm_f32", [
            Ptr("X"), Ptr("scale"), Ptr("B"), Ptr("in_mean"), Ptr("in_var"), Ptr("Y"), X.shape[0], X.shape[1],
            prod(X.shape[2:]), eps, Stream()])


@op_implementation(op="MatMulInteger", name=IMPLEMENTATION_NAME)
class MI355XMatMulInteger(ONNXForward):
    """8-bit x 8-bit -> int32 on int8 MFMA, bit-exact against the ONNX formula in 64-bit integers (parity with the
    reference unpinned: it has no implementation of its own); operands int8 or uint8 (independently), zero
    points read on the device: absent, one value, one per row of A or one per column of B. A may be
    a stack of matrices against a 2-D B (the stack is folded into M). The reference can only run this
    node through ONNX Runtime (onnx_op.py:686-687)."""

    @staticmethod
    def _plan(node, state, sdfg):
        A = in_desc_with_name(node, state, sdfg, "A")
        B = in_desc_with_name(node, state, sdfg, "B")
        Y = out_desc_with_name(node, state, sdfg, "Y")
        eight_bit = (dace.int8, dace.uint8)
        if A.dtype not in eight_bit or B.dtype not in eight_bit or Y.dtype != dace.int32:
            return None
        if len(A.shape) < 2 or len(B.shape) != 2 or A.shape[-1] != B.shape[0]:
            return None
        M, K, N = prod(A.shape[:-1]), A.shape[-1], B.shape[1]
        if tuple(Y.shape) != tuple(A.shape[:-1]) + (N, ) or not _contig(A, B, Y):
            return None
        counts = {}
        for zp, operand, full in (("a_zero_point", A, M), ("b_zero_point", B, N)):
            counts[zp] = 1
            if not _has_input(node, state, zp):
                continue
            d = in_desc_with_name(node, state, sdfg, zp)
            if d.dtype != operand.dtype or not _contig(d):
                return None
            if d.total_size == 1:
                continue
            # one per row of A: [M] for a matrix, [D1, ..., M, 1] for a stack; one per column of B: [N]
            shape = tuple(d.shape)
            per_row = shape == (A.shape[0], ) if len(A.shape) == 2 else shape == tuple(A.shape[:-1]) + (1, )
            if not (per_row if zp == "a_zero_point" else shape == (N, )):
                return None
            counts[zp] = full
        return M, N, K, A.dtype == dace.uint8, B.dtype == dace.uint8, counts["a_zero_point"], counts["b_zero_point"]

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        return MI355XMatMulInteger._plan(node, state, sdfg) is not None

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        M, N, K, a_unsigned, b_unsigned, za_count, zb_count = MI355XMatMulInteger._plan(node, state, sdfg)
        za = "a_zero_point" if _has_input(node, state, "a_zero_point") else None
        zb = "b_zero_point" if _has_input(node, state, "b_zero_point") else None
        return kernel_call_for_node(node, state, "mi355x_matmul_integer", [
            Ptr("A"), Ptr("B"), Ptr(za), Ptr(zb), Ptr("Y"), M, N, K, int(a_unsigned), int(b_unsigned), za_count, zb_count,
            Stream()])


# ------------------------------------------------------------------------------------
# row reductions


@op_implementation(op="Softmax", name=IMPLEMENTATION_NAME)
class MI355XSoftmax(ONNXForward):
    """Softmax along ``node.axis`` only, the semantics of PureSoftmax
    (:352-364; for the last axis this equals the opset-11 flattened form)."""

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        X = in_desc_with_name(node, state, sdfg, "input")
        Y = out_desc_with_name(node, state, sdfg, "output")
        if not _is_f32(X, Y) or not _contig(X, Y) or tuple(X.shape) != tuple(Y.shape):
            return False
        return len(X.shape) >= 1 and -len(X.shape) <= node.axis < len(X.shape)

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        X = in_desc_with_name(node, state, sdfg, "input")
        axis = node.axis % len(X.shape)
        outer, axis_len, inner = prod(X.shape[:axis]), X.shape[axis], prod(X.shape[axis + 1:])
        return kernel_call_for_node(node, state, "mi355x_softmax_f32",
                                    [Ptr("input"), Ptr("output"), outer, axis_len, inner, Stream()])


@op_implementation(op="LogSoftmax", name=IMPLEMENTATION_NAME)
class MI355XLogSoftmax(ONNXForward):
    """LogSoftmax along ``node.axis`` only, as PureLogSoftmax computes it (:594-616), in one pass."""

    forward_can_be_applied = MI355XSoftmax.forward_can_be_applied

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        X = in_desc_with_name(node, state, sdfg, "input")
        axis = node.axis % len(X.shape)
        outer, axis_len, inner = prod(X.shape[:axis]), X.shape[axis], prod(X.shape[axis + 1:])
        return kernel_call_for_node(node, state, "mi355x_log_softmax_f32",
                                    [Ptr("input"), Ptr("output"), outer, axis_len, inner, Stream()])


@op_implementation(op="FusedAttention", name=IMPLEMENTATION_NAME)
class MI355XFusedAttention(ONNXForward):
    """``softmax(scale * Q K^T) V`` in one launch; scores stay in registers. The
    operands are the arrays on the edges or the (shape, strides, offset) views the
    fusion pass attached (``_q_view`` ... ``_o_view``): head split / merge of a
    [B, S, H*D] projection is addressing, not a copy."""

    SUPPORTED_HEAD = 64   #: head size of the kernel; 128 keys run in one pass, any other number in blocks of 128

    @staticmethod
    def supports(plan) -> bool:
        return plan is not None and plan[3] >= 1 and plan[4] == MI355XFusedAttention.SUPPORTED_HEAD

    @staticmethod
    def _operands(node, state, sdfg):
        out = []
        for conn, attr, getter in (("Q", "_q_view", in_desc_with_name), ("K", "_k_view", in_desc_with_name),
                                   ("V", "_v_view", in_desc_with_name), ("O", "_o_view", out_desc_with_name)):
            d = getter(node, state, sdfg, conn)
            view = getattr(node, attr, None)
            out.append((dace.Array(d.dtype, view[0], view[1]) if view else d, int(view[2]) if view and len(view) > 2 else 0))
        return out

    @staticmethod
    def _plan(descs):
        """(batch0, batch1, Sq, Sk, D, [strides of Q, K, V, O as {b0, b1, row}]) or None."""
        (Q, _), (K, _), (V, _), (O, _) = descs
        if not _is_f32(Q, K, V, O) or min(len(d.shape) for d in (Q, K, V, O)) < 2:
            return None
        batch = tuple(Q.shape[:-2])
        if any(tuple(d.shape[:-2]) != batch for d in (K, V, O)) or len([e for e in batch if e != 1]) > 2:
            return None
        (Sq, D), (Sk, D2) = Q.shape[-2:], K.shape[-2:]
        if D2 != D or tuple(V.shape[-2:]) != (Sk, D) or tuple(O.shape[-2:]) != (Sq, D):
            return None
        if any(d.strides[-1] != 1 for d in (Q, K, V, O)):
            return None
        if any(st % 4 or st < 0 for d in (Q, K, V, O) for st, e in zip(d.strides[:-1], d.shape[:-1]) if e != 1):
            return None
        dims = [i for i, e in enumerate(batch) if e != 1]
        dims = [None] * (2 - len(dims)) + dims
        ext = [1 if i is None else batch[i] for i in dims]
        strides = [[0 if i is None else d.strides[i] for i in dims] + [d.strides[-2]] for d in (Q, K, V, O)]
        return ext[0], ext[1], Sq, Sk, D, strides

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        plan = MI355XFusedAttention._plan(MI355XFusedAttention._operands(node, state, sdfg))
        return MI355XFusedAttention.supports(plan)

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        descs = MI355XFusedAttention._operands(node, state, sdfg)
        b0, b1, Sq, Sk, D, strides = MI355XFusedAttention._plan(descs)
        offs = [o for _, o in descs]
        return kernel_call_for_node(node, state, "mi355x_attention_f32", [
            Ptr("Q", offs[0]), Ptr("K", offs[1]), Ptr("V", offs[2]), Ptr("O", offs[3]), b0, b1, Sq, Sk, D,
            I64Array(strides[0]), I64Array(strides[1]), I64Array(strides[2]), I64Array(strides[3]),
            float(node.scale if node.scale is not None else 1.0), Stream()])


def _reduce_split(node, X):
    """(outer, axis_len, inner, reduced axes) when the reduced axes are adjacent -- which makes them one axis
    of the product length -- or None."""
    rank = len(X.shape)
    axes = sorted(a % rank for a in node.axes) if node.axes is not None else list(range(rank))
    if not axes or axes != list(range(axes[0], axes[-1] + 1)) or any(not -rank <= a < rank for a in (node.axes or [])):
        return None
    return prod(X.shape[:axes[0]]), prod(X.shape[axes[0]:axes[-1] + 1]), prod(X.shape[axes[-1] + 1:]), axes


def _reduce_axes(node, X):
    """Sorted, normalised reduced axes (all of them when the attribute is absent), or None when invalid."""
    rank = len(X.shape)
    if node.axes is None:
        return list(range(rank))
    if any(not -rank <= a < rank for a in node.axes) or len({a % rank for a in node.axes}) != len(node.axes):
        return None
    return sorted(a % rank for a in node.axes)


def _reduce_impl(op_name, kind, cite):
    @op_implementation(op=op_name, name=IMPLEMENTATION_NAME)
    class Impl(ONNXForward):
        __doc__ = (f"{op_name} over ``axes`` (attribute form, opset < 13 / 18): adjacent axes as one axis of the "
                   f"product length, any other set through the general kernel ({cite}).")

        @staticmethod
        def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
            X = in_desc_with_name(node, state, sdfg, "data")
            Y = out_desc_with_name(node, state, sdfg, "reduced")
            if not _is_f32(X, Y) or not _contig(X, Y) or not 1 <= len(X.shape) <= MAX_ELTWISE_DIMS:
                return False
            axes = _reduce_axes(node, X)
            if not axes or prod([X.shape[a] for a in axes]) < 1:
                return False
            keep = node.keepdims is None or bool(node.keepdims)
            want = [1 if d in axes else e for d, e in enumerate(X.shape)] if keep else \
                [e for d, e in enumerate(X.shape) if d not in axes]
            return [e for e in Y.shape if e != 1] == [e for e in want if e != 1] and \
                Y.total_size == prod([e for d, e in enumerate(X.shape) if d not in axes])

        @staticmethod
        def forward(node, state: SDFGState, sdfg: SDFG):
            X = in_desc_with_name(node, state, sdfg, "data")
            split = _reduce_split(node, X)
            if split is None:       # the reduced axes are not adjacent
                axes = _reduce_axes(node, X)
                return kernel_call_for_node(node, state, "mi355x_reduce_nd_f32", [
                    kind, Ptr("data"), Ptr("reduced"), len(X.shape), I64Array(X.shape), I64Array(X.strides),
                    I64Array([int(d in axes) for d in range(len(X.shape))]), Stream()])
            outer, axis_len, inner, _ = split
            if kind == _lib.REDUCE_MEAN:
                return kernel_call_for_node(node, state, "mi355x_reduce_mean_f32",
                                            [Ptr("data"), Ptr("reduced"), outer, axis_len, inner, Stream()])
            return kernel_call_for_node(node, state, "mi355x_reduce_f32",
                                        [kind, Ptr("data"), Ptr("reduced"), outer, axis_len, inner, Stream()])

    Impl.__name__ = Impl.__qualname__ = "MI355X" + op_name
    return Impl


MI355XReduceMean = _reduce_impl("ReduceMean", _lib.REDUCE_MEAN, "PureReduceMean, :97-109")
MI355XReduceSum = _reduce_impl("ReduceSum", _lib.REDUCE_SUM, "PureReduceSum, :301-313")
MI355XReduceMax = _reduce_impl("ReduceMax", _lib.REDUCE_MAX, "PureReduceMax, :316-328")
MI355XReduceMin = _reduce_impl("ReduceMin", _lib.REDUCE_MIN, "PureReduceMin, :331-343")


@op_implementation(op="LayerNormalization", name=IMPLEMENTATION_NAME)
class MI355XLayerNormalization(ONNXForward):
    """One-pass layer normalization over the dimensions from ``axis`` on."""

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        X = in_desc_with_name(node, state, sdfg, "X")
        S = in_desc_with_name(node, state, sdfg, "Scale")
        Y = out_desc_with_name(node, state, sdfg, "Y")
        descs = [X, S, Y]
        if _has_input(node, state, "B"):
            descs.append(in_desc_with_name(node, state, sdfg, "B"))
        if not _is_f32(*descs) or not _contig(*descs) or tuple(X.shape) != tuple(Y.shape):
            return False
        if _has_output(node, state, "Mean") or _has_output(node, state, "InvStdDev"):
            return False
        if len(X.shape) < 1 or not (-len(X.shape) <= node.axis < len(X.shape)):
            return False
        cols = prod(X.shape[node.axis % len(X.shape):])
        return all(d.total_size == cols for d in descs[1:2] + descs[3:])

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        X = in_desc_with_name(node, state, sdfg, "X")
        axis = node.axis % len(X.shape)
        rows, cols = prod(X.shape[:axis]), prod(X.shape[axis:])
        beta = "B" if _has_input(node, state, "B") else None
        return kernel_call_for_node(node, state, "mi355x_layernorm_f32", [
            Ptr("X"), Ptr("Scale"), Ptr(beta), Ptr("Y"), rows, cols, float(node.epsilon), Stream()])


# ------------------------------------------------------------------------------------
# elementwise


def _binary_impl(op_name, opcode, conns=("A", "B", "C")):
    a_conn, b_conn, c_conn = conns

    @op_implementation(op=op_name, name=IMPLEMENTATION_NAME)
    class Impl(ONNXForward):
        __doc__ = f"``{c_conn} = {a_conn} {op_name.lower()} {b_conn}`` with numpy broadcasting, one pass."

        @staticmethod
        def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
            A = in_desc_with_name(node, state, sdfg, a_conn)
            B = in_desc_with_name(node, state, sdfg, b_conn)
            C = out_desc_with_name(node, state, sdfg, c_conn)
            if not _is_f32(A, B, C) or not _contig(C):
                return False
            out = _broadcast_shape(A.shape, B.shape)
            return out is not None and tuple(C.shape) == out and len(out) <= MAX_ELTWISE_DIMS

        @staticmethod
        def forward(node, state: SDFGState, sdfg: SDFG):
            A = in_desc_with_name(node, state, sdfg, a_conn)
            B = in_desc_with_name(node, state, sdfg, b_conn)
            C = out_desc_with_name(node, state, sdfg, c_conn)
            return kernel_call_for_node(node, state, "mi355x_eltwise_f32", [
                opcode, Ptr(a_conn), Ptr(b_conn), Ptr(c_conn), len(C.shape), I64Array(C.shape),
                I64Array(_broadcast_strides(A, C.shape)), I64Array(_broadcast_strides(B, C.shape)), Stream()])

    Impl.__name__ = Impl.__qualname__ = "MI355X" + op_name
    return Impl


MI355XAdd = _binary_impl("Add", _lib.OP_ADD)
MI355XSub = _binary_impl("Sub", _lib.OP_SUB)
MI355XMul = _binary_impl("Mul", _lib.OP_MUL)
MI355XDiv = _binary_impl("Div", _lib.OP_DIV)
# PurePow (pure_implementations.py:59-74) special-cases the exponent 2 of the exported LayerNorm; so does the kernel
MI355XPow = _binary_impl("Pow", _lib.OP_POW, conns=("X", "Y", "Z"))


def _unary_impl(op_name, opcode, in_conn, out_conn, extra_check=None):
    @op_implementation(op=op_name, name=IMPLEMENTATION_NAME)
    class Impl(ONNXForward):
        __doc__ = f"Elementwise {op_name}, one pass, 16 bytes per lane."

        @staticmethod
        def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
            X = in_desc_with_name(node, state, sdfg, in_conn)
            Y = out_desc_with_name(node, state, sdfg, out_conn)
            if not _is_f32(X, Y) or not _contig(X, Y) or tuple(X.shape) != tuple(Y.shape):
                return False
            return extra_check(node) if extra_check else True

        @staticmethod
        def forward(node, state: SDFGState, sdfg: SDFG):
            X = in_desc_with_name(node, state, sdfg, in_conn)
            return kernel_call_for_node(node, state, "mi355x_eltwise_f32", [
                opcode, Ptr(in_conn), None, Ptr(out_conn), 1, I64Array([X.total_size]), I64Array([1]),
                None, Stream()])

    Impl.__name__ = Impl.__qualname__ = "MI355X" + op_name
    return Impl


MI355XRelu = _unary_impl("Relu", _lib.OP_RELU, "X", "Y")
MI355XGelu = _unary_impl("Gelu", _lib.OP_GELU, "X", "Y",
                         extra_check=lambda node: (node.approximate or "none") == "none")
MI355XErf = _unary_impl("Erf", _lib.OP_ERF, "input", "output")
MI355XSqrt = _unary_impl("Sqrt", _lib.OP_SQRT, "X", "Y")
# PureLog (:23-38), Tanh (:296-298), PureSigmoid (:701-712), Softplus (:696-698), PureReciprocal (:275-293);
# Exp, Neg and Abs have no pure expansion in the reference
MI355XLog = _unary_impl("Log", _lib.OP_LOG, "input", "output")
MI355XTanh = _unary_impl("Tanh", _lib.OP_TANH, "input", "output")
MI355XExp = _unary_impl("Exp", _lib.OP_EXP, "input", "output")
MI355XSigmoid = _unary_impl("Sigmoid", _lib.OP_SIGMOID, "X", "Y")
MI355XSoftplus = _unary_impl("Softplus", _lib.OP_SOFTPLUS, "X", "Y")
MI355XReciprocal = _unary_impl("Reciprocal", _lib.OP_RECIPROCAL, "X", "Y")
MI355XNeg = _unary_impl("Neg", _lib.OP_NEG, "X", "Y")
MI355XAbs = _unary_impl("Abs", _lib.OP_ABS, "X", "Y")


# ------------------------------------------------------------------------------------
# data movement


@op_implementation(op="Transpose", name=IMPLEMENTATION_NAME)
class MI355XTranspose(ONNXForward):
    """Permutation copy for 4-byte element types."""

    @staticmethod
    def _perm(node, rank):
        return list(node.perm) if node.perm is not None else list(reversed(range(rank)))

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        X = in_desc_with_name(node, state, sdfg, "data")
        Y = out_desc_with_name(node, state, sdfg, "transposed")
        if X.dtype != Y.dtype or X.dtype.bytes != 4 or not _contig(Y) or len(X.shape) > MAX_ELTWISE_DIMS:
            return False
        perm = MI355XTranspose._perm(node, len(X.shape))
        if sorted(perm) != list(range(len(X.shape))):
            return False
        return tuple(Y.shape) == tuple(X.shape[p] for p in perm)

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        X = in_desc_with_name(node, state, sdfg, "data")
        perm = MI355XTranspose._perm(node, len(X.shape))
        return kernel_call_for_node(node, state, "mi355x_permute_b32", [
            Ptr("data"), Ptr("transposed"), len(perm), I64Array([X.shape[p] for p in perm]),
            I64Array([X.strides[p] for p in perm]), Stream()])


# ONNX TensorProto data types the cast kernel converts between (the values of Cast's ``to``)
_CAST_TYPES = {"float32": 1, "uint8": 2, "int8": 3, "int32": 6, "int64": 7, "bool_": 9, "float64": 11}


@op_implementation(op="Cast", name=IMPLEMENTATION_NAME)
class MI355XCast(ONNXForward):
    """Elementwise conversion in one pass (PureCast, :382-430: a map of ``__output = __input``)."""

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        X = in_desc_with_name(node, state, sdfg, "input")
        Y = out_desc_with_name(node, state, sdfg, "output")
        return X.dtype.name in _CAST_TYPES and Y.dtype.name in _CAST_TYPES and _contig(X, Y) and \
            tuple(X.shape) == tuple(Y.shape) and (node.to is None or int(node.to) == _CAST_TYPES[Y.dtype.name])

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        X = in_desc_with_name(node, state, sdfg, "input")
        Y = out_desc_with_name(node, state, sdfg, "output")
        return kernel_call_for_node(node, state, "mi355x_cast", [
            Ptr("input"), _CAST_TYPES[X.dtype.name], Ptr("output"), _CAST_TYPES[Y.dtype.name], int(X.total_size), Stream()])


@op_implementation(op="Slice", name=IMPLEMENTATION_NAME)
class MI355XSlice(ONNXForward):
    """Slice with constant ``starts`` / ``ends`` / ``axes`` / ``steps`` as one strided gather of 4-byte
    elements: any axes, any non-zero steps. PureSlice (:619-693) covers axis 0 with step 1 and explicit
    ``axes`` and ``steps`` only and leaves the rest to ONNX Runtime."""

    @staticmethod
    def _ranges(node, state, sdfg):
        """slice_ranges(...) of the node, or None when an index input is not a constant."""
        from ...onnx.shape_inference import slice_ranges, ShapeInferenceError
        model = getattr(sdfg, "_parent_onnx_model", None)
        idx = []
        for name in ("starts", "ends", "axes", "steps"):
            if not _has_input(node, state, name):
                idx.append(None)
                continue
            edge = [e for e in state.in_edges(node) if e.dst_conn == name][0]
            if state.in_edges(edge.src):
                return None             # computed by another node
            if model is not None and edge.src.data in model.clean_weights:
                idx.append([int(v) for v in model.clean_weights[edge.src.data].detach().cpu().reshape(-1).tolist()])
            elif edge.src.data in getattr(sdfg, "_constant_inputs", {}):       # the call form donnx.ONNXSlice(...)
                idx.append([int(v) for v in sdfg._constant_inputs[edge.src.data].reshape(-1)])
            else:
                return None
        if idx[0] is None or idx[1] is None:
            return None
        try:
            return slice_ranges(in_desc_with_name(node, state, sdfg, "data").shape, *idx)
        except ShapeInferenceError:
            return None

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        X = in_desc_with_name(node, state, sdfg, "data")
        Y = out_desc_with_name(node, state, sdfg, "output")
        if X.dtype != Y.dtype or X.dtype.bytes != 4 or not _contig(X, Y) or not 1 <= len(X.shape) <= MAX_ELTWISE_DIMS:
            return False
        ranges = MI355XSlice._ranges(node, state, sdfg)
        return ranges is not None and tuple(Y.shape) == tuple(c for _, _, c in ranges)

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        X = in_desc_with_name(node, state, sdfg, "data")
        ranges = MI355XSlice._ranges(node, state, sdfg)
        offset = sum(first * stride for (first, _, count), stride in zip(ranges, X.strides)) if all(c for _, _, c in ranges) else 0
        return kernel_call_for_node(node, state, "mi355x_permute_b32", [
            Ptr("data", offset), Ptr("output"), len(ranges), I64Array([c for _, _, c in ranges]),
            I64Array([stride * step for (_, step, _), stride in zip(ranges, X.strides)]), Stream()])


def _alias_impl(op_name, in_conn, out_conn):
    @op_implementation(op=op_name, name=IMPLEMENTATION_NAME)
    class Impl(ONNXForward):
        __doc__ = (f"{op_name} of contiguous data is a view: the output aliases the input's storage. "
                   "(PureReshape copies through ``np.reshape``, pure_implementations.py:496-513; "
                   "like it, the constant ``shape`` input is dropped.)")

        @staticmethod
        def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
            X = in_desc_with_name(node, state, sdfg, in_conn)
            Y = out_desc_with_name(node, state, sdfg, out_conn)
            return X.dtype == Y.dtype and _contig(X, Y) and X.total_size == Y.total_size

        @staticmethod
        def forward(node, state: SDFGState, sdfg: SDFG):
            return AliasNode(node.label + "_view", in_conn, out_conn)

    Impl.__name__ = Impl.__qualname__ = "MI355X" + op_name
    return Impl


MI355XReshape = _alias_impl("Reshape", "data", "reshaped")
MI355XFlatten = _alias_impl("Flatten", "input", "output")
MI355XIdentity = _alias_impl("Identity", "input", "output")
# Squeeze / Unsqueeze have no pure expansion in the reference (ONNX Runtime copies the data there)
MI355XSqueeze = _alias_impl("Squeeze", "data", "squeezed")
MI355XUnsqueeze = _alias_impl("Unsqueeze", "data", "expanded")


@op_implementation(op="Pad", name=IMPLEMENTATION_NAME)
class MI355XPad(ONNXForward):
    """No kernel of its own: a constant zero Pad of the spatial axes is folded into the Conv that reads
    it before expansion (``transformation/fusion.py``, the reference's ``PadConvFusion``). A Pad that is
    still in the graph at expansion time is refused, which the reference would hand to ONNX Runtime."""

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        return False

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        raise NotImplementedError("Pad is only supported folded into a Conv")


@op_implementation(op="FusedElementwise", name=IMPLEMENTATION_NAME)
class MI355XFusedElementwise(ONNXForward):
    """A group of elementwise nodes merged by the fusion pass: one launch of the program kernel. Inputs
    ``X__i`` are tensors of the output's shape (``kinds[i] == 1``) or vectors along the last axis (2)."""

    @staticmethod
    def _inputs(node, state, sdfg):
        conns = sorted((c for c in node.in_connectors if c.startswith("X__")), key=lambda c: int(c[3:]))
        kinds = list(node.kinds or [])
        return conns, kinds

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        conns, kinds = MI355XFusedElementwise._inputs(node, state, sdfg)
        Y = out_desc_with_name(node, state, sdfg, "Y")
        if len(conns) != len(kinds) or not conns or not _is_f32(Y) or not Y.is_contiguous() or not node.program:
            return False
        for c, k in zip(conns, kinds):
            d = in_desc_with_name(node, state, sdfg, c)
            if not _is_f32(d) or not d.is_contiguous():
                return False
            if k == _lib.PROGRAM_TENSOR and tuple(d.shape) != tuple(Y.shape):
                return False
            if k == _lib.PROGRAM_VECTOR and (not Y.shape or d.total_size != Y.shape[-1]):
                return False
        return kinds.count(_lib.PROGRAM_TENSOR) <= _lib.PROGRAM_MAX_TENSORS and \
            kinds.count(_lib.PROGRAM_VECTOR) <= _lib.PROGRAM_MAX_VECTORS and \
            len(node.program) <= _lib.PROGRAM_MAX_INSTR and len(node.immediates or []) <= _lib.PROGRAM_MAX_IMM

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        conns, kinds = MI355XFusedElementwise._inputs(node, state, sdfg)
        Y = out_desc_with_name(node, state, sdfg, "Y")
        tensors = [c for c, k in zip(conns, kinds) if k == _lib.PROGRAM_TENSOR]
        vectors = [c for c, k in zip(conns, kinds) if k == _lib.PROGRAM_VECTOR]
        imms = list(node.immediates or [])
        return kernel_call_for_node(node, state, "mi355x_eltwise_program_f32", [
            PtrArray(tensors), len(tensors), PtrArray(vectors), len(vectors), Ptr("Y"), int(Y.total_size),
            int(Y.shape[-1]) if Y.shape else 1, U32Array(node.program), len(node.program), F32Array(imms), len(imms), Stream()])



@op_implementation(op="Sum", name=IMPLEMENTATION_NAME)
class MI355XSum(ONNXForward):
    """Sum of up to four tensors of one shape -- the case PureSum accepts (:529-591, all shapes equal to the
    output's) -- as one launch of the program kernel: every input read once, no intermediate sums."""

    @staticmethod
    def _inputs(node):
        return sorted((c for c in node.in_connectors if c.startswith("data_0__")), key=lambda c: int(c[len("data_0__"):]))

    @staticmethod
    def forward_can_be_applied(node, state: SDFGState, sdfg: SDFG) -> bool:
        conns = MI355XSum._inputs(node)
        Y = out_desc_with_name(node, state, sdfg, "sum")
        if not 1 <= len(conns) <= _lib.PROGRAM_MAX_TENSORS or not _is_f32(Y) or not _contig(Y):
            return False
        descs = [in_desc_with_name(node, state, sdfg, c) for c in conns]
        return all(_is_f32(d) and _contig(d) and tuple(d.shape) == tuple(Y.shape) for d in descs)

    @staticmethod
    def forward(node, state: SDFGState, sdfg: SDFG):
        conns = MI355XSum._inputs(node)
        Y = out_desc_with_name(node, state, sdfg, "sum")
        tensor = lambda i: (_lib.PROGRAM_TENSOR << 6) | i
        if len(conns) == 1:
            program = [_lib.OP_COPY | tensor(0) << 16]
        else:   # r0 = t0 + t1; r0 = r0 + t2; ...
            program = [_lib.OP_ADD | tensor(0) << 16 | tensor(1) << 24]
            program += [_lib.OP_ADD | (_lib.PROGRAM_REG << 6) << 16 | tensor(i) << 24 for i in range(2, len(conns))]
        return kernel_call_for_node(node, state, "mi355x_eltwise_program_f32", [
            PtrArray(conns), len(conns), PtrArray([]), 0, Ptr("sum"), int(Y.total_size),
            int(Y.shape[-1]) if Y.shape else 1, U32Array(program), len(program), F32Array([]), 0, Stream()])

"""Graph-level fusion of ONNX library nodes before expansion.

The reference fuses at graph level too, with pattern transformations over the
SDFG: ``PadConvFusion`` folds a Pad into the Conv that follows
(``daceml/transformation/pad_conv_fusion.py:13-95``), ``TaskletFusion`` merges
elementwise tasklets (``tasklet_fusion.py:35``), ``ReshapeElimination`` drops
Reshapes. Here the patterns are the ones that remove HBM round trips around a
contraction, because the MFMA kernels can absorb them:

===========================================  =====================================
pattern (every intermediate single-use)      becomes
===========================================  =====================================
MatMul -> Div/Mul by a constant scalar       MatMul with ``_alpha``
MatMul -> Add(1-D bias over N)               MatMul with input connector ``_bias``
MatMul/Gemm -> Relu | Gelu                   ``_activation``
MatMul -> Add(tensor of the output's shape)  input connector ``_residual``
Conv -> Relu                                 ``_activation = "relu"``
X -> Reshape/Transpose chain -> MatMul       MatMul reads X through ``_a_view`` /
                                             ``_b_view`` (shape, strides)
MatMul with a constant [K, N] weight         weight copied once as [N, K];
                                             ``_b_view`` strides [1, K]
MatMul -> Transpose -> Reshape               MatMul writes the final array through
                                             ``_y_view``
ReduceMean, Sub, Pow(2), ReduceMean,         LayerNormalization (what exporters below
Add(eps), Sqrt, Div, Mul(gamma), Add(beta)   opset 17 write for ``nn.LayerNorm``)
Div(sqrt 2), Erf, Add(1), Mul(x), Mul(0.5)   Gelu (exact erf form, any operand order)
Pad(constant 0, spatial) -> Conv             the Conv's ``pads`` grow (``PadConvFusion``)
MatMul(alpha) -> Softmax(last) -> MatMul     FusedAttention when the kernel supports the
                                             shape (head size 64)
MatMuls of one A with constant weights       one MatMul with the weights (and biases)
(the Q, K, V projections)                    concatenated along N; the readers
                                             address their slice of the wide result
                                             through (shape, strides, offset) views
===========================================  =====================================

The annotations are private attributes / connectors (leading underscore) that
the ``"mi355x"`` MatMul, Gemm and Conv expansions understand; the reference
passes per-node tuning the same way (``node._algorithm``,
``cudnn_implementations.py:251-254``). Order inside the kernel epilogue is fixed:
alpha, bias, activation, residual -- a pattern is only folded when it respects it.
Nodes left without consumers are removed afterwards.
"""
import logging
import typing

import numpy as np

from .. import _lib

from ..sdfg import SDFG, SDFGState, AccessNode, Array, _contiguous_strides

log = logging.getLogger(__name__)


# ----------------------------------------------------------------------------- graph helpers
def _is_op(node, *names):
    schema = getattr(node, "schema", None)
    return schema is not None and schema.name in names


def _in_edge(state, node, conn):
    c = [e for e in state.in_edges(node) if e.dst_conn == conn]
    return c[0] if len(c) == 1 else None


def _out_edge(state, node, conn):
    c = [e for e in state.out_edges(node) if e.src_conn == conn]
    return c[0] if len(c) == 1 else None


def _single_consumer(sdfg, state, access: AccessNode):
    """The only reader of a transient that is written once; None otherwise."""
    desc = sdfg.arrays[access.data]
    if not desc.transient or len(state.in_edges(access)) != 1:
        return None
    outs = state.out_edges(access)
    if len(outs) != 1:
        return None
    # no other access node of the same array may read it
    for n in state.nodes():
        if isinstance(n, AccessNode) and n is not access and n.data == access.data:
            return None
    return outs[0]


def _producer(state, access: AccessNode):
    ins = state.in_edges(access)
    return ins[0] if len(ins) == 1 else None


def _constant_value(sdfg, name) -> typing.Optional[np.ndarray]:
    model = getattr(sdfg, "_parent_onnx_model", None)
    if model is None:
        return None
    w = model.clean_weights.get(name)
    return None if w is None else w.detach().cpu().numpy()


def _reshape_strides(shape, strides, new_shape):
    """Strides that view (shape, strides) as ``new_shape`` without copying, or None
    (the no-copy reshape rule of numpy)."""
    old = [(s, st) for s, st in zip(shape, strides) if s != 1]
    new_strides = [0] * len(new_shape)
    oi = 0
    ni = 0
    while ni < len(new_shape):
        if new_shape[ni] == 1:
            new_strides[ni] = 0
            ni += 1
            continue
        if oi >= len(old):
            return None
        # grow a group of old dims and a group of new dims until their sizes match
        o_size, n_size = old[oi][0], new_shape[ni]
        o_end, n_end = oi + 1, ni + 1
        while o_size != n_size:
            if o_size < n_size:
                if o_end >= len(old):
                    return None
                o_size *= old[o_end][0]
                o_end += 1
            else:
                while n_end < len(new_shape) and new_shape[n_end] == 1:
                    n_end += 1
                if n_end >= len(new_shape):
                    return None
                n_size *= new_shape[n_end]
                n_end += 1
        # the old group must be contiguous within itself
        for k in range(oi, o_end - 1):
            if old[k][1] != old[k + 1][1] * old[k + 1][0]:
                return None
        st = old[o_end - 1][1]
        for k in range(n_end - 1, ni - 1, -1):
            new_strides[k] = st if new_shape[k] != 1 else 0
            st *= new_shape[k]
        oi, ni = o_end, n_end
    if oi != len(old):
        return None
    return new_strides


# ----------------------------------------------------------------------------- elementwise folds
def _replace_output(sdfg, state, node, out_conn, folded_node, folded_out_conn):
    """``node`` takes over the output of ``folded_node``; the intermediate array and
    ``folded_node`` disappear."""
    mid_edge = _out_edge(state, node, out_conn)
    mid_access = mid_edge.dst
    final_edge = _out_edge(state, folded_node, folded_out_conn)
    state.remove_edge(mid_edge)
    state.add_edge(node, out_conn, final_edge.dst, None, final_edge.data)
    state.remove_node(folded_node)
    state.remove_node(mid_access)
    del sdfg.arrays[mid_access.data]


def _fuse_pad_conv(sdfg: SDFG, state: SDFGState) -> int:
    """A constant zero ``Pad`` of the spatial axes whose only reader is a ``Conv`` becomes part of the
    convolution's ``pads`` (the reference's ``PadConvFusion``, ``daceml/transformation/pad_conv_fusion.py``:
    constant mode, value 0, 4-D, eight constant pads, nothing padded along batch or channels)."""
    fused = 0
    for pad in list(state.nodes()):
        if not _is_op(pad, "Pad") or (pad.mode or "constant") != "constant":
            continue
        out_e, data_e, pads_e = _out_edge(state, pad, "output"), _in_edge(state, pad, "data"), _in_edge(state, pad, "pads")
        if out_e is None or data_e is None or pads_e is None or not isinstance(out_e.dst, AccessNode):
            continue
        use = _single_consumer(sdfg, state, out_e.dst)
        if use is None or not _is_op(use.dst, "Conv") or use.dst_conn != "X" or len(sdfg.arrays[out_e.dst.data].shape) != 4:
            continue
        conv = use.dst
        pads = _constant_value(sdfg, pads_e.src.data)
        value_e = _in_edge(state, pad, "constant_value")
        value = _constant_value(sdfg, value_e.src.data) if value_e is not None else np.zeros(1)
        if pads is None or pads.size != 8 or value is None or value.size != 1 or float(value.reshape(-1)[0]) != 0.0:
            continue
        pads = [int(v) for v in pads.reshape(-1)]
        if any(pads[i] != 0 for i in (0, 1, 4, 5)) or min(pads) < 0:
            continue
        if (conv.auto_pad or "NOTSET") != "NOTSET":
            continue
        old = list(conv.pads) if conv.pads is not None else [0, 0, 0, 0]
        conv.pads = [old[0] + pads[2], old[1] + pads[3], old[2] + pads[6], old[3] + pads[7]]
        mid = out_e.dst
        state.remove_edge(use)
        state.add_edge(data_e.src, None, conv, "X", sdfg.make_array_memlet(data_e.src.data))
        state.remove_node(pad)
        state.remove_node(mid)
        del sdfg.arrays[mid.data]
        fused += 1
    return fused


def _fold_batchnorm_into_conv(sdfg: SDFG, state: SDFGState) -> int:
    """Conv with constant weights whose only reader is an inference ``BatchNormalization`` with constant
    parameters: the per-channel affine map moves into the convolution, ``W'[oc] = W[oc] * a[oc]`` and
    ``bias' = (bias - mean) * a + B`` with ``a = scale / sqrt(var + eps)``, computed once at graph-preparation
    time (the folded copies are new weights; the originals stay untouched). The reference has no counterpart:
    its BatchNormalization expansion is the training form (``img_op_implementations.py:329-407``) and an
    exported eval() network runs this pair as two ONNX Runtime nodes."""
    model = getattr(sdfg, "_parent_onnx_model", None)
    if model is None:
        return 0
    import torch
    from ..onnx.onnx_importer import clean_onnx_name
    by_clean = {clean_onnx_name(k): k for k in model.weights}

    def constant(node, conn):
        e = _in_edge(state, node, conn)
        if e is None or not isinstance(e.src, AccessNode) or e.src.data not in by_clean or state.in_edges(e.src):
            return None
        w = model.weights[by_clean[e.src.data]]
        return (e, w) if w.dtype == torch.float32 else None

    folded = 0
    for conv in list(state.nodes()):
        if not _is_op(conv, "Conv") or _in_edge(state, conv, "_residual") is not None or getattr(conv, "_activation", None):
            continue
        y_e = _out_edge(state, conv, "Y")
        if y_e is None or not isinstance(y_e.dst, AccessNode):
            continue
        use = _single_consumer(sdfg, state, y_e.dst)
        if use is None or not _is_op(use.dst, "BatchNormalization") or use.dst_conn != "X":
            continue
        bn = use.dst
        if len(state.out_edges(bn)) != 1 or _out_edge(state, bn, "Y") is None:
            continue        # training outputs present
        w = constant(conv, "W")
        params = [constant(bn, c) for c in ("scale", "B", "in_mean", "in_var")]
        has_bias = _in_edge(state, conv, "B") is not None
        bias = constant(conv, "B") if has_bias else None
        if w is None or any(p is None for p in params) or (has_bias and bias is None):
            continue
        oc = w[1].shape[0]
        if any(tuple(p[1].shape) != (oc, ) for p in params) or (bias is not None and tuple(bias[1].shape) != (oc, )):
            continue
        eps = 1e-5 if bn.epsilon is None else float(bn.epsilon)
        scale, beta, mean, var = (p[1].double() for p in params)
        a = scale / torch.sqrt(var + eps)
        new_w = (w[1].double() * a.reshape(-1, *([1] * (w[1].dim() - 1)))).float().contiguous()
        new_b = (((bias[1].double() if bias is not None else torch.zeros_like(mean)) - mean) * a + beta).float().contiguous()
        w_name, b_name = by_clean[w[0].src.data] + "_bnfold_" + bn.label, by_clean[w[0].src.data] + "_bnfold_bias_" + bn.label
        model.weights[w_name], model.weights[b_name] = new_w, new_b
        w_clean, b_clean = clean_onnx_name(w_name), clean_onnx_name(b_name)
        sdfg.add_array(w_clean, list(new_w.shape), sdfg.arrays[w[0].src.data].dtype, transient=False)
        sdfg.add_array(b_clean, [oc], sdfg.arrays[w[0].src.data].dtype, transient=False)
        state.remove_edge(w[0])
        state.add_edge(state.add_access(w_clean), None, conv, "W", sdfg.make_array_memlet(w_clean))
        if bias is not None:
            state.remove_edge(bias[0])
        else:
            conv.add_in_connector("B")
        state.add_edge(state.add_access(b_clean), None, conv, "B", sdfg.make_array_memlet(b_clean))
        out_e = _out_edge(state, bn, "Y")
        mid = y_e.dst
        state.remove_edge(y_e)
        state.add_edge(conv, "Y", out_e.dst, None, sdfg.make_array_memlet(out_e.dst.data))
        state.remove_node(bn)
        state.remove_node(mid)
        del sdfg.arrays[mid.data]
        folded += 1
    return folded


def _fold_into_contractions(sdfg: SDFG, state: SDFGState) -> int:
    folded = 0
    changed = True
    while changed:
        changed = False
        for node in state.nodes():
            if not _is_op(node, "MatMul", "Gemm", "Conv"):
                continue
            out_e = _out_edge(state, node, "Y")
            if out_e is None or not isinstance(out_e.dst, AccessNode):
                continue
            use = _single_consumer(sdfg, state, out_e.dst)
            if use is None:
                continue
            nxt = use.dst
            ydesc = sdfg.arrays[out_e.dst.data]
            has_bias = _in_edge(state, node, "_bias") is not None
            has_res = _in_edge(state, node, "_residual") is not None
            act = getattr(node, "_activation", None)

            # ---- scalar scale -> alpha (must come first in the epilogue)
            if _is_op(node, "MatMul") and _is_op(nxt, "Div", "Mul") and use.dst_conn == "A" \
                    and not (has_bias or has_res or act):
                other = _in_edge(state, nxt, "B")
                val = _constant_value(sdfg, other.src.data) if other is not None else None
                if val is not None and val.size == 1 and tuple(sdfg.arrays[_out_edge(state, nxt, "C").dst.data].shape) == tuple(ydesc.shape):
                    v = float(val.reshape(-1)[0])
                    node._alpha = getattr(node, "_alpha", 1.0) * ((1.0 / v) if _is_op(nxt, "Div") else v)
                    _replace_output(sdfg, state, node, "Y", nxt, "C")
                    folded += 1
                    changed = True
                    break
            # ---- bias over the last dimension
            if _is_op(node, "MatMul") and _is_op(nxt, "Add") and not (has_bias or has_res or act):
                other_conn = "B" if use.dst_conn == "A" else "A"
                other = _in_edge(state, nxt, other_conn)
                if other is not None:
                    od = sdfg.arrays[other.src.data]
                    n_dim = ydesc.shape[-1]
                    out_shape = tuple(sdfg.arrays[_out_edge(state, nxt, "C").dst.data].shape)
                    if od.total_size == n_dim and od.shape and od.shape[-1] == n_dim and od.is_contiguous() \
                            and out_shape == tuple(ydesc.shape) and n_dim > 1:
                        node.add_in_connector("_bias")
                        state.add_edge(other.src, None, node, "_bias", other.data)
                        _replace_output(sdfg, state, node, "Y", nxt, "C")
                        folded += 1
                        changed = True
                        break
            # ---- activation (it runs before the residual in the epilogue: a Gemm whose C is a full [M, N]
            # addend, which the expansion passes as the residual, cannot take one)
            if _is_op(node, "Gemm") and _in_edge(state, node, "C") is not None:
                c_shape = tuple(sdfg.arrays[_in_edge(state, node, "C").src.data].shape)
                has_res = has_res or not (len(c_shape) == 1 or (len(c_shape) == 2 and c_shape[0] == 1))
            if _is_op(nxt, "Relu", "Gelu") and not has_res and act is None:
                is_gelu = _is_op(nxt, "Gelu")
                if (not is_gelu or ((nxt.approximate or "none") == "none" and not _is_op(node, "Conv"))):
                    node._activation = "gelu" if is_gelu else "relu"
                    _replace_output(sdfg, state, node, "Y", nxt, "Y")
                    folded += 1
                    changed = True
                    break
            # ---- convolution: the Relu after the residual (the end of a ResNet block)
            if _is_op(node, "Conv") and has_res and _is_op(nxt, "Relu") and getattr(node, "_activation_after", None) is None:
                node._activation_after = "relu"
                _replace_output(sdfg, state, node, "Y", nxt, "Y")
                folded += 1
                changed = True
                break
            # ---- residual (after bias and activation in the epilogue)
            if _is_op(node, "MatMul", "Conv") and _is_op(nxt, "Add") and not has_res:
                other_conn = "B" if use.dst_conn == "A" else "A"
                other = _in_edge(state, nxt, other_conn)
                if other is not None:
                    od = sdfg.arrays[other.src.data]
                    out_shape = tuple(sdfg.arrays[_out_edge(state, nxt, "C").dst.data].shape)
                    if tuple(od.shape) == tuple(ydesc.shape) == out_shape and od.is_contiguous() and ydesc.is_contiguous():
                        node.add_in_connector("_residual")
                        state.add_edge(other.src, None, node, "_residual", other.data)
                        _replace_output(sdfg, state, node, "Y", nxt, "C")
                        folded += 1
                        changed = True
                        break
    return folded


def _fold_operand_scale(sdfg: SDFG, state: SDFGState) -> int:
    """``Mul`` / ``Div`` of a MatMul operand by a scalar constant (``nn.MultiheadAttention`` scales the
    queries before ``Q K^T``) moves into the node's alpha: (c A) B = c (A B). The scaled tensor must have
    the MatMul as its only reader."""
    folded = 0
    changed = True
    while changed:
        changed = False
        for node in state.nodes():
            if not _is_op(node, "MatMul"):
                continue
            for conn in ("A", "B"):
                e = _in_edge(state, node, conn)
                if e is None or not isinstance(e.src, AccessNode) or _single_consumer(sdfg, state, e.src) is None:
                    continue
                prod = _producer(state, e.src)
                if prod is None or not _is_op(prod.src, "Mul", "Div"):
                    continue
                scale = prod.src
                # the constant may be either factor of a Mul, only the divisor of a Div
                for c_conn, x_conn in (("B", "A"), ("A", "B")) if _is_op(scale, "Mul") else (("B", "A"), ):
                    c_e, x_e = _in_edge(state, scale, c_conn), _in_edge(state, scale, x_conn)
                    if c_e is None or x_e is None or not isinstance(x_e.src, AccessNode):
                        continue
                    val = _constant_value(sdfg, c_e.src.data)
                    if val is None or val.size != 1 or \
                            tuple(sdfg.arrays[x_e.src.data].shape) != tuple(sdfg.arrays[e.src.data].shape):
                        continue
                    v = float(val.reshape(-1)[0])
                    node._alpha = getattr(node, "_alpha", 1.0) * ((1.0 / v) if _is_op(scale, "Div") else v)
                    mid = e.src
                    state.remove_edge(e)
                    state.add_edge(x_e.src, None, node, conn, sdfg.make_array_memlet(x_e.src.data))
                    state.remove_node(scale)
                    state.remove_node(mid)
                    del sdfg.arrays[mid.data]
                    folded += 1
                    changed = True
                    break
                if changed:
                    break
            if changed:
                break
    return folded


# ----------------------------------------------------------------------------- view folds
def _input_view(sdfg, state, access: AccessNode):
    """Walk back through Reshape/Transpose producers of ``access``. Returns
    (source access node, shape, strides) describing ``access`` as a strided view
    of the source array, or None when there is nothing to fold."""
    chain = []
    cur = access
    while True:
        prod = _producer(state, cur)
        if prod is None or not sdfg.arrays[cur.data].transient:
            break
        n = prod.src
        if _is_op(n, "Transpose"):
            chain.append(("T", n))
            cur = _in_edge(state, n, "data").src
        elif _is_op(n, "Reshape", "Squeeze", "Unsqueeze"):     # all three: the same elements under another shape
            chain.append(("R", n))
            cur = _in_edge(state, n, "data").src
        else:
            break
        if not isinstance(cur, AccessNode):
            return None
    if not chain:
        return None
    src = sdfg.arrays[cur.data]
    if not src.is_contiguous():
        return None
    shape, strides = list(src.shape), list(src.strides)
    for kind, n in reversed(chain):
        if kind == "T":
            perm = list(n.perm) if n.perm is not None else list(reversed(range(len(shape))))
            shape, strides = [shape[p] for p in perm], [strides[p] for p in perm]
        else:
            new_shape = list(sdfg.arrays[_out_edge(state, n, n.schema.outputs[0].name).dst.data].shape)
            new_strides = _reshape_strides(shape, strides, new_shape)
            if new_strides is None:
                return None
            shape, strides = new_shape, new_strides
    if tuple(shape) != tuple(sdfg.arrays[access.data].shape):
        return None
    return cur, shape, strides


def _fold_views(sdfg: SDFG, state: SDFGState) -> int:
    from ..onnx.op_implementations.mi355x_implementations import _BatchPlan
    folded = 0
    for node in state.nodes():
        if not _is_op(node, "MatMul"):
            continue
        a_e, b_e, y_e = _in_edge(state, node, "A"), _in_edge(state, node, "B"), _out_edge(state, node, "Y")
        if a_e is None or b_e is None or y_e is None:
            continue

        def desc_of(edge, view):
            d = sdfg.arrays[edge.data.data]
            return Array(d.dtype, view[0], view[1]) if view else d

        views = {"A": getattr(node, "_a_view", None), "B": getattr(node, "_b_view", None),
                 "Y": getattr(node, "_y_view", None)}
        # ---- inputs: read through Reshape/Transpose chains
        for conn, edge, attr in (("A", a_e, "_a_view"), ("B", b_e, "_b_view")):
            if views[conn] is not None or not isinstance(edge.src, AccessNode):
                continue
            found = _input_view(sdfg, state, edge.src)
            if found is None:
                continue
            src_access, shape, strides = found
            trial = dict(views)
            trial[conn] = (shape, strides)
            plan = _BatchPlan(Array(sdfg.arrays[src_access.data].dtype, trial["A"][0], trial["A"][1]) if trial["A"] else sdfg.arrays[a_e.data.data],
                              Array(sdfg.arrays[src_access.data].dtype, trial["B"][0], trial["B"][1]) if trial["B"] else sdfg.arrays[b_e.data.data],
                              desc_of(y_e, trial["Y"]))
            if not plan.ok:
                continue
            state.remove_edge(edge)
            new_edge = state.add_edge(src_access, None, node, conn, sdfg.make_array_memlet(src_access.data))
            setattr(node, attr, (shape, strides))
            views[conn] = (shape, strides)
            if conn == "A":
                a_e = new_edge
            else:
                b_e = new_edge
            folded += 1
        # ---- output: write through Transpose (-> Reshape)
        if views["Y"] is None and _in_edge(state, node, "_bias") is None and _in_edge(state, node, "_residual") is None \
                and getattr(node, "_activation", None) is None and isinstance(y_e.dst, AccessNode):
            use = _single_consumer(sdfg, state, y_e.dst)
            if use is not None and _is_op(use.dst, "Transpose"):
                tnode = use.dst
                ydesc = sdfg.arrays[y_e.dst.data]
                perm = list(tnode.perm) if tnode.perm is not None else list(reversed(range(len(ydesc.shape))))
                t_access = _out_edge(state, tnode, "transposed").dst
                t_strides = _contiguous_strides(sdfg.arrays[t_access.data].shape)
                y_strides = [0] * len(perm)
                for k, p in enumerate(perm):
                    y_strides[p] = t_strides[k]
                final_access, drop = t_access, [tnode]
                use2 = _single_consumer(sdfg, state, t_access)
                if use2 is not None and _is_op(use2.dst, "Reshape") and use2.dst_conn == "data":
                    final_access = _out_edge(state, use2.dst, "reshaped").dst
                    drop.append(use2.dst)
                if ydesc.is_contiguous() and sdfg.arrays[final_access.data].is_contiguous() and y_strides[-1] == 1:
                    view = (list(ydesc.shape), y_strides)
                    plan = _BatchPlan(desc_of(a_e, views["A"]), desc_of(b_e, views["B"]), Array(ydesc.dtype, view[0], view[1]))
                    if plan.ok:
                        mids = [y_e.dst] + ([t_access] if final_access is not t_access else [])
                        state.remove_edge(y_e)
                        state.add_edge(node, "Y", final_access, None, sdfg.make_array_memlet(final_access.data))
                        for d in drop:
                            state.remove_node(d)
                        for m in mids:
                            state.remove_node(m)
                            del sdfg.arrays[m.data]
                        node._y_view = view
                        folded += 1
    return folded


def _pretranspose_weights(sdfg: SDFG, state: SDFGState) -> int:
    """MatMul with a constant 2-D B ([K, N], n-contiguous as ONNX stores it): keep a
    second copy of the weight laid out [N, K] and let the node read it through a
    ``_b_view`` of shape [K, N] with strides [1, K]. With both operands contiguous
    along k every MFMA fragment is a 16-byte LDS / global access (the layout
    PyTorch's ``nn.Linear`` and ONNX ``Gemm(transB=1)`` use anyway). Done once, at
    graph-preparation time -- the analogue of the reference's constant folding
    (``daceml/transformation/constant_folding.py:48``)."""
    model = getattr(sdfg, "_parent_onnx_model", None)
    if model is None:
        return 0
    from ..onnx.onnx_importer import clean_onnx_name
    by_clean = {clean_onnx_name(k): k for k in model.weights}
    done = 0
    for node in state.nodes():
        if not _is_op(node, "MatMul") or getattr(node, "_b_view", None) is not None:
            continue
        b_e = _in_edge(state, node, "B")
        if b_e is None or not isinstance(b_e.src, AccessNode) or b_e.src.data not in by_clean:
            continue
        if state.in_edges(b_e.src):  # written inside the graph: not a constant
            continue
        desc = sdfg.arrays[b_e.src.data]
        if len(desc.shape) != 2 or not desc.is_contiguous() or desc.dtype.name != "float32":
            continue
        k, n = desc.shape
        if k % 4 or n % 4:
            continue
        t_name = b_e.src.data + "_kcontig"
        if t_name not in sdfg.arrays:
            sdfg.add_array(t_name, [n, k], desc.dtype, transient=False)
            model.weights[by_clean[b_e.src.data] + "_kcontig"] = model.weights[by_clean[b_e.src.data]].t().contiguous()
        t_access = None
        for cand in state.nodes():
            if isinstance(cand, AccessNode) and cand.data == t_name:
                t_access = cand
        if t_access is None:
            t_access = state.add_access(t_name)
        state.remove_edge(b_e)
        state.add_edge(t_access, None, node, "B", sdfg.make_array_memlet(t_name))
        node._b_view = ([k, n], [1, k])
        done += 1
    return done


# ----------------------------------------------------------------------------- decomposed operators
def _other_input(state, node, edge):
    """The edge into the other operand of a binary node (connectors A and B)."""
    return _in_edge(state, node, "B" if edge.dst_conn == "A" else "A")


def _scalar_constant(sdfg, edge) -> typing.Optional[float]:
    if edge is None or not isinstance(edge.src, AccessNode):
        return None
    val = _constant_value(sdfg, edge.src.data)
    return float(val.reshape(-1)[0]) if val is not None and val.size == 1 else None


def _next_op(sdfg, state, access, *ops):
    """The single reader of ``access`` if it is one of ``ops`` and ``access`` is a
    transient written once; else None."""
    use = _single_consumer(sdfg, state, access)
    return use if use is not None and _is_op(use.dst, *ops) else None


def _out_access(state, node, conn):
    e = _out_edge(state, node, conn)
    return e.dst if e is not None and isinstance(e.dst, AccessNode) else None


def _drop_chain(sdfg, state, nodes, keep_access):
    """Remove ``nodes`` and the transients only they touched (never ``keep_access``)."""
    touched = []
    for n in nodes:
        for e in state.in_edges(n) + state.out_edges(n):
            a = e.src if e.dst is n else e.dst
            if isinstance(a, AccessNode) and a not in touched:
                touched.append(a)
        state.remove_node(n)
    for a in touched:
        if a in keep_access:
            continue
        if not state.in_edges(a) and not state.out_edges(a):
            state.remove_node(a)
            desc = sdfg.arrays.get(a.data)
            still_used = any(isinstance(n, AccessNode) and n.data == a.data for n in state.nodes())
            if desc is not None and desc.transient and not still_used:
                del sdfg.arrays[a.data]


def _fuse_decomposed_layernorm(sdfg: SDFG, state: SDFGState) -> int:
    """ReduceMean(x) -> Sub(x, mean) -> Pow(.,2) -> ReduceMean -> Add(eps) -> Sqrt ->
    Div(centred, std) -> Mul(gamma) [-> Add(beta)], over the last axis, becomes one
    LayerNormalization node. This is the decomposition the reference executes node
    by node (pure_implementations.py:97-109, 82-84, 59-74, 77-79, 41-56, 92-94)."""
    from ..onnx.nodes.onnx_op import get_onnx_node
    fused = 0
    for m1 in list(state.nodes()):
        if m1 not in state.nodes() or not _is_op(m1, "ReduceMean"):
            continue
        x_e = _in_edge(state, m1, "data")
        mean = _out_access(state, m1, "reduced")
        if x_e is None or mean is None or not isinstance(x_e.src, AccessNode):
            continue
        xdesc = sdfg.arrays[x_e.src.data]
        rank = len(xdesc.shape)
        last_axis = lambda n: n.axes is not None and [a % rank for a in n.axes] == [rank - 1] and \
            (n.keepdims is None or bool(n.keepdims))
        if rank < 1 or not last_axis(m1) or not xdesc.is_contiguous():
            continue
        sub_use = _next_op(sdfg, state, mean, "Sub")
        if sub_use is None or sub_use.dst_conn != "B":
            continue
        sub = sub_use.dst
        if _in_edge(state, sub, "A").src.data != x_e.src.data:
            continue
        centred = _out_access(state, sub, "C")
        if centred is None or not sdfg.arrays[centred.data].transient or len(state.in_edges(centred)) != 1:
            continue
        readers = state.out_edges(centred)
        pow_e = [e for e in readers if _is_op(e.dst, "Pow") and e.dst_conn == "X"]
        div_e = [e for e in readers if _is_op(e.dst, "Div") and e.dst_conn == "A"]
        if len(readers) != 2 or len(pow_e) != 1 or len(div_e) != 1:
            continue
        pw, div = pow_e[0].dst, div_e[0].dst
        if _scalar_constant(sdfg, _in_edge(state, pw, "Y")) != 2.0:
            continue
        sq = _out_access(state, pw, "Z")
        m2_use = _next_op(sdfg, state, sq, "ReduceMean") if sq is not None else None
        if m2_use is None or not last_axis(m2_use.dst):
            continue
        m2 = m2_use.dst
        var = _out_access(state, m2, "reduced")
        add_use = _next_op(sdfg, state, var, "Add") if var is not None else None
        if add_use is None:
            continue
        add_eps = add_use.dst
        eps = _scalar_constant(sdfg, _other_input(state, add_eps, add_use))
        var_eps = _out_access(state, add_eps, "C")
        sqrt_use = _next_op(sdfg, state, var_eps, "Sqrt") if var_eps is not None and eps is not None else None
        if sqrt_use is None:
            continue
        sqrt = sqrt_use.dst
        std = _out_access(state, sqrt, "Y")
        std_use = _next_op(sdfg, state, std, "Div") if std is not None else None
        if std_use is None or std_use.dst is not div or std_use.dst_conn != "B":
            continue
        normed = _out_access(state, div, "C")
        mul_use = _next_op(sdfg, state, normed, "Mul") if normed is not None else None
        if mul_use is None:
            continue
        mul = mul_use.dst
        gamma_e = _other_input(state, mul, mul_use)
        cols = xdesc.shape[-1]

        def is_row_vector(e):
            if e is None or not isinstance(e.src, AccessNode):
                return False
            d = sdfg.arrays[e.src.data]
            return d.total_size == cols and d.shape and d.shape[-1] == cols and d.is_contiguous()

        if not is_row_vector(gamma_e):
            continue
        out = _out_access(state, mul, "C")
        if out is None or tuple(sdfg.arrays[out.data].shape) != tuple(xdesc.shape):
            continue
        chain = [m1, sub, pw, m2, add_eps, sqrt, div, mul]
        beta_e = None
        add_use2 = _next_op(sdfg, state, out, "Add")
        if add_use2 is not None and is_row_vector(_other_input(state, add_use2.dst, add_use2)):
            out2 = _out_access(state, add_use2.dst, "C")
            if out2 is not None and tuple(sdfg.arrays[out2.data].shape) == tuple(xdesc.shape):
                beta_e = _other_input(state, add_use2.dst, add_use2)
                chain.append(add_use2.dst)
                out = out2
        if not sdfg.arrays[out.data].is_contiguous():
            continue
        ln = get_onnx_node("LayerNormalization")(m1.label + "_layernorm", axis=-1, epsilon=eps)
        state.add_node(ln)
        ln.add_in_connector("X")
        state.add_edge(x_e.src, None, ln, "X", sdfg.make_array_memlet(x_e.src.data))
        ln.add_in_connector("Scale")
        state.add_edge(gamma_e.src, None, ln, "Scale", sdfg.make_array_memlet(gamma_e.src.data))
        if beta_e is not None:
            ln.add_in_connector("B")
            state.add_edge(beta_e.src, None, ln, "B", sdfg.make_array_memlet(beta_e.src.data))
        ln.add_out_connector("Y")
        keep = [x_e.src, gamma_e.src, out] + ([beta_e.src] if beta_e is not None else [])
        _drop_chain(sdfg, state, chain, keep)
        state.add_edge(ln, "Y", out, None, sdfg.make_array_memlet(out.data))
        fused += 1
    return fused


def _fuse_decomposed_gelu(sdfg: SDFG, state: SDFGState) -> int:
    """x / sqrt(2) (or x * 1/sqrt(2)) -> Erf -> + 1 -> * x -> * 0.5, with the last two
    multiplications in either order, becomes one Gelu node."""
    from ..onnx.nodes.onnx_op import get_onnx_node
    fused = 0
    for erf in list(state.nodes()):
        if erf not in state.nodes() or not _is_op(erf, "Erf"):
            continue
        scaled_e = _in_edge(state, erf, "input")
        if scaled_e is None or not isinstance(scaled_e.src, AccessNode) or _single_consumer(sdfg, state, scaled_e.src) is None:
            continue
        prod_e = _producer(state, scaled_e.src)
        if prod_e is None or not _is_op(prod_e.src, "Div", "Mul"):
            continue
        scale = prod_e.src
        a_e, b_e = _in_edge(state, scale, "A"), _in_edge(state, scale, "B")
        if _is_op(scale, "Div"):
            x_e, c = a_e, _scalar_constant(sdfg, b_e)
            ok = c is not None and abs(c - 2.0 ** 0.5) < 1e-4
        else:
            ca, cb = _scalar_constant(sdfg, a_e), _scalar_constant(sdfg, b_e)
            x_e, c = (b_e, ca) if ca is not None else (a_e, cb)
            ok = c is not None and abs(c - 0.5 ** 0.5) < 1e-4
        if not ok or x_e is None or not isinstance(x_e.src, AccessNode):
            continue
        x_name = x_e.src.data
        erf_out = _out_access(state, erf, "output")
        add_use = _next_op(sdfg, state, erf_out, "Add") if erf_out is not None else None
        if add_use is None or _scalar_constant(sdfg, _other_input(state, add_use.dst, add_use)) != 1.0:
            continue
        add1 = add_use.dst
        cur = _out_access(state, add1, "C")
        chain, seen_x, seen_half = [scale, erf, add1], False, False
        for _ in range(2):  # the two multiplications, either order
            mul_use = _next_op(sdfg, state, cur, "Mul") if cur is not None else None
            if mul_use is None:
                break
            other = _other_input(state, mul_use.dst, mul_use)
            if other is None or not isinstance(other.src, AccessNode):
                break
            if not seen_x and other.src.data == x_name:
                seen_x = True
            elif not seen_half and _scalar_constant(sdfg, other) == 0.5:
                seen_half = True
            else:
                break
            chain.append(mul_use.dst)
            cur = _out_access(state, mul_use.dst, "C")
        # 0.5 may also have been applied to x before the product: x * 0.5 * (1 + erf) is not matched here
        if not (seen_x and seen_half) or cur is None:
            continue
        xdesc, ydesc = sdfg.arrays[x_name], sdfg.arrays[cur.data]
        if tuple(xdesc.shape) != tuple(ydesc.shape) or not xdesc.is_contiguous() or not ydesc.is_contiguous():
            continue
        gelu = get_onnx_node("Gelu")(erf.label + "_gelu")
        state.add_node(gelu)
        gelu.add_in_connector("X")
        state.add_edge(x_e.src, None, gelu, "X", sdfg.make_array_memlet(x_name))
        gelu.add_out_connector("Y")
        _drop_chain(sdfg, state, chain, [x_e.src, cur])
        state.add_edge(gelu, "Y", cur, None, sdfg.make_array_memlet(cur.data))
        fused += 1
    return fused


# ----------------------------------------------------------------------------- attention
def _fuse_attention(sdfg: SDFG, state: SDFGState) -> int:
    """scores = alpha * (Q K^T); probs = Softmax(scores, last axis); ctx = probs V, every
    intermediate single-use, becomes one FusedAttention node that reads Q, K, V and
    writes ctx through the views the two MatMuls already carry. Runs after the view
    folds (so K^T and the head split are strides) and before the projections are
    widened (which only rebases those views)."""
    from ..onnx.nodes.onnx_op import get_onnx_node
    from ..onnx.op_implementations.mi355x_implementations import MI355XFusedAttention
    fused = 0
    for sm in list(state.nodes()):
        if sm not in state.nodes() or not _is_op(sm, "Softmax"):
            continue
        s_in, probs = _in_edge(state, sm, "input"), _out_access(state, sm, "output")
        if s_in is None or probs is None or not isinstance(s_in.src, AccessNode):
            continue
        scores = s_in.src
        rank = len(sdfg.arrays[scores.data].shape)
        if rank < 2 or sm.axis % rank != rank - 1 or _single_consumer(sdfg, state, scores) is None:
            continue
        prod1 = _producer(state, scores)
        use2 = _next_op(sdfg, state, probs, "MatMul")
        if prod1 is None or not _is_op(prod1.src, "MatMul") or use2 is None or use2.dst_conn != "A":
            continue
        mm1, mm2 = prod1.src, use2.dst
        if any(_in_edge(state, n, c) is not None for n in (mm1, mm2) for c in ("_bias", "_residual")) \
                or any(getattr(n, "_activation", None) for n in (mm1, mm2)) \
                or getattr(mm1, "_y_view", None) or getattr(mm2, "_a_view", None) or getattr(mm2, "_alpha", 1.0) != 1.0:
            continue
        q_e, kt_e, v_e, o_e = _in_edge(state, mm1, "A"), _in_edge(state, mm1, "B"), _in_edge(state, mm2, "B"), \
            _out_edge(state, mm2, "Y")
        if None in (q_e, kt_e, v_e, o_e) or not all(isinstance(e.src, AccessNode) for e in (q_e, kt_e, v_e)):
            continue

        def view_of(edge, node, attr):
            v = getattr(node, attr, None)
            if v:
                return [list(v[0]), list(v[1]), int(v[2]) if len(v) > 2 else 0]
            d = sdfg.arrays[edge.data.data]
            return [list(d.shape), list(d.strides), 0]

        qv, ktv = view_of(q_e, mm1, "_a_view"), view_of(kt_e, mm1, "_b_view")
        vv, ov = view_of(v_e, mm2, "_b_view"), view_of(o_e, mm2, "_y_view")
        if len(ktv[0]) < 2:
            continue
        kv = [ktv[0][:-2] + [ktv[0][-1], ktv[0][-2]], ktv[1][:-2] + [ktv[1][-1], ktv[1][-2]], ktv[2]]  # K = (K^T)^T
        f32 = sdfg.arrays[q_e.data.data].dtype
        plan = MI355XFusedAttention._plan([(Array(f32, v[0], v[1]), v[2]) for v in (qv, kv, vv, ov)])
        if not MI355XFusedAttention.supports(plan):
            continue
        node = get_onnx_node("FusedAttention")(mm1.label + "_attention", scale=float(getattr(mm1, "_alpha", 1.0)))
        state.add_node(node)
        for conn, edge, view in (("Q", q_e, qv), ("K", kt_e, kv), ("V", v_e, vv)):
            node.add_in_connector(conn)
            state.add_edge(edge.src, None, node, conn, sdfg.make_array_memlet(edge.src.data))
            setattr(node, "_" + conn.lower() + "_view", tuple(view))
        node.add_out_connector("O")
        node._o_view = tuple(ov)
        out_access = o_e.dst
        _drop_chain(sdfg, state, [mm1, sm, mm2], [q_e.src, kt_e.src, v_e.src, out_access])
        state.add_edge(node, "O", out_access, None, sdfg.make_array_memlet(out_access.data))
        fused += 1
    return fused


# ----------------------------------------------------------------------------- horizontal fusion
def _rebase_strides(shape, strides, n_old, n_new):
    """A view (shape, strides) into a contiguous [rows, n_old] array, re-expressed
    for the same elements inside a [rows, n_new] array (n_new >= n_old, same column
    positions). Dimensions that step whole rows scale by n_new / n_old; dimensions
    that step inside a row keep their stride. None if a dimension does neither."""
    out, inside = [], 0
    for extent, st in zip(shape, strides):
        if extent == 1 or st == 0:
            out.append(st)
        elif st % n_old == 0:
            out.append(st // n_old * n_new)
        else:
            inside += (extent - 1) * st
            out.append(st)
    return out if inside < n_old else None


def _fuse_shared_input_matmuls(sdfg: SDFG, state: SDFGState) -> int:
    """MatMul nodes that multiply the same A by different constant [K, N_i] weights
    (or, all of them, by [N_i, K] weights read through a folded Transpose, the form
    ``nn.Linear`` exports to; optionally each with a fused 1-D bias) become one MatMul
    against the weights concatenated along N. Applies when every reader of every Y_i is a MatMul
    operand, because only the GEMM can address a column slice of the wide result
    without a copy. One launch instead of len(group), and A is read once."""
    import torch
    from ..onnx.onnx_importer import clean_onnx_name
    from ..onnx.op_implementations.mi355x_implementations import _BatchPlan
    model = getattr(sdfg, "_parent_onnx_model", None)
    if model is None:
        return 0
    by_clean = {clean_onnx_name(k): k for k in model.weights}

    def constant_input(node, conn, ndim):
        e = _in_edge(state, node, conn)
        if e is None or not isinstance(e.src, AccessNode) or e.src.data not in by_clean or state.in_edges(e.src):
            return None
        d = sdfg.arrays[e.src.data]
        if len(d.shape) != ndim or not d.is_contiguous() or d.dtype.name != "float32":
            return None
        return e

    groups = {}
    for node in state.nodes():
        if not _is_op(node, "MatMul"):
            continue
        if any(getattr(node, a, None) is not None for a in ("_a_view", "_y_view", "_activation")) \
                or getattr(node, "_alpha", 1.0) != 1.0 or _in_edge(state, node, "_residual") is not None:
            continue
        a_e, y_e = _in_edge(state, node, "A"), _out_edge(state, node, "Y")
        b_e = constant_input(node, "B", 2)
        if a_e is None or b_e is None or y_e is None or not isinstance(a_e.src, AccessNode) \
                or not isinstance(y_e.dst, AccessNode):
            continue
        # B either as ONNX stores it ([K, N]) or as nn.Linear does ([N, K] read through a folded Transpose)
        b_view, transposed = getattr(node, "_b_view", None), False
        if b_view is not None:
            n_w, k_w = sdfg.arrays[b_e.src.data].shape
            if list(b_view[0]) != [k_w, n_w] or list(b_view[1]) != [1, k_w] or (len(b_view) > 2 and b_view[2]):
                continue
            transposed = True
        has_bias = _in_edge(state, node, "_bias") is not None
        bias_e = constant_input(node, "_bias", 1) if has_bias else None
        if has_bias and bias_e is None:
            continue
        ydesc = sdfg.arrays[y_e.dst.data]
        if not ydesc.transient or not ydesc.is_contiguous() or len(state.in_edges(y_e.dst)) != 1:
            continue
        if any(isinstance(n, AccessNode) and n is not y_e.dst and n.data == y_e.dst.data for n in state.nodes()):
            continue
        readers = state.out_edges(y_e.dst)
        if not readers or not all((_is_op(r.dst, "MatMul") and r.dst_conn in ("A", "B")) or
                                  (_is_op(r.dst, "FusedAttention") and r.dst_conn in ("Q", "K", "V")) for r in readers):
            continue
        if any(r.dst is node for r in readers):
            continue
        k, width = sdfg.arrays[b_e.src.data].shape[::-1] if transposed else sdfg.arrays[b_e.src.data].shape
        a_writes = sum(len(state.in_edges(n)) for n in state.nodes() if isinstance(n, AccessNode) and n.data == a_e.src.data)
        if a_writes > 1:
            continue
        groups.setdefault((a_e.src.data, k, has_bias, transposed), []).append((node, a_e, b_e, bias_e, y_e, readers, width))

    fused = 0
    for (_, k_total, _, transposed), members in groups.items():
        if len(members) < 2:
            continue
        # a reader of one member's output must not be another member (they all run at once)
        nodes = [m[0] for m in members]
        if any(r.dst in nodes for m in members for r in m[5]):
            continue
        widths = [m[6] for m in members]
        if any(w % 4 for w in widths):
            continue
        n_total = sum(widths)
        first = members[0]
        y0 = sdfg.arrays[first[4].dst.data]
        wide_shape = list(y0.shape[:-1]) + [n_total]
        if any(list(sdfg.arrays[m[4].dst.data].shape[:-1]) != wide_shape[:-1] for m in members):
            continue
        # ---- new views of every reader; give up on the whole group if one cannot be expressed
        rewires, start, ok = [], 0, True
        for (node, a_e, b_e, bias_e, y_e, readers, _), width in zip(members, widths):
            ydesc = sdfg.arrays[y_e.dst.data]
            for r in readers:
                attr = {"A": "_a_view", "B": "_b_view", "Q": "_q_view", "K": "_k_view", "V": "_v_view"}[r.dst_conn]
                old = getattr(r.dst, attr, None)
                shape, strides = (old[0], old[1]) if old else (list(ydesc.shape), list(ydesc.strides))
                offset = old[2] if old and len(old) > 2 else 0
                new_strides = _rebase_strides(shape, strides, width, n_total)
                if new_strides is None or offset != 0:
                    ok = False
                    break
                rewires.append((r, attr, (list(shape), new_strides, start)))
            start += width
        if not ok:
            continue
        trial = {}
        for r, attr, view in rewires:
            trial.setdefault(r.dst, {})[attr] = view
        for consumer, views in trial.items():
            if _is_op(consumer, "FusedAttention"):
                from ..onnx.op_implementations.mi355x_implementations import MI355XFusedAttention
                cur = [views.get(a, getattr(consumer, a)) for a in ("_q_view", "_k_view", "_v_view", "_o_view")]
                plan = MI355XFusedAttention._plan([(Array(y0.dtype, v[0], v[1]), v[2]) for v in cur])
                if not MI355XFusedAttention.supports(plan):
                    ok = False
                continue

            def operand(conn, attr):
                v = views.get(attr, getattr(consumer, attr, None))
                if v:
                    return Array(y0.dtype, v[0], v[1])
                e = _in_edge(state, consumer, conn)
                return sdfg.arrays[e.data.data]
            yv = getattr(consumer, "_y_view", None)
            yd = Array(y0.dtype, yv[0], yv[1]) if yv else sdfg.arrays[_out_edge(state, consumer, "Y").data.data]
            if not _BatchPlan(operand("A", "_a_view"), operand("B", "_b_view"), yd).ok:
                ok = False
        if not ok:
            continue
        # ---- constants: weights [K, sum N_i], biases [sum N_i]
        w_name = by_clean[first[2].src.data] + "_hcat"
        model.weights[w_name] = torch.cat([model.weights[by_clean[m[2].src.data]] for m in members],
                                          dim=0 if transposed else 1).contiguous()
        w_clean = clean_onnx_name(w_name)
        sdfg.add_array(w_clean, list(model.weights[w_name].shape), y0.dtype, transient=False)
        b_clean = None
        if first[3] is not None:
            b_name = by_clean[first[3].src.data] + "_hcat"
            model.weights[b_name] = torch.cat([model.weights[by_clean[m[3].src.data]].reshape(-1) for m in members]).contiguous()
            b_clean = clean_onnx_name(b_name)
            sdfg.add_array(b_clean, [n_total], y0.dtype, transient=False)
        wide = first[4].dst.data + "_hcat"
        sdfg.add_transient(wide, wide_shape, y0.dtype)
        wide_access = state.add_access(wide)
        # ---- the first member becomes the wide MatMul
        keep = first[0]
        state.remove_edge(first[2])
        state.add_edge(state.add_access(w_clean), None, keep, "B", sdfg.make_array_memlet(w_clean))
        if transposed:
            keep._b_view = ([k_total, n_total], [1, k_total])
        if b_clean is not None:
            state.remove_edge(first[3])
            state.add_edge(state.add_access(b_clean), None, keep, "_bias", sdfg.make_array_memlet(b_clean))
        state.remove_edge(first[4])
        state.add_edge(keep, "Y", wide_access, None, sdfg.make_array_memlet(wide))
        for r, attr, view in rewires:
            state.remove_edge(r)
            state.add_edge(wide_access, None, r.dst, r.dst_conn, sdfg.make_array_memlet(wide))
            setattr(r.dst, attr, view)
        for node, a_e, b_e, bias_e, y_e, readers, _ in members:
            if node is not keep:
                state.remove_node(node)
            state.remove_node(y_e.dst)
            del sdfg.arrays[y_e.dst.data]
        fused += len(members) - 1
    return fused


_EW_BINARY = {"Add": _lib.OP_ADD, "Sub": _lib.OP_SUB, "Mul": _lib.OP_MUL, "Div": _lib.OP_DIV, "Pow": _lib.OP_POW}
_EW_UNARY = {"Relu": _lib.OP_RELU, "Gelu": _lib.OP_GELU, "Erf": _lib.OP_ERF, "Sqrt": _lib.OP_SQRT, "Identity": _lib.OP_COPY,
             "Log": _lib.OP_LOG, "Tanh": _lib.OP_TANH, "Sigmoid": _lib.OP_SIGMOID, "Softplus": _lib.OP_SOFTPLUS,
             "Reciprocal": _lib.OP_RECIPROCAL, "Exp": _lib.OP_EXP, "Neg": _lib.OP_NEG, "Abs": _lib.OP_ABS}


def _fuse_elementwise(sdfg: SDFG, state: SDFGState) -> int:
    """Groups of elementwise nodes (Add, Sub, Mul, Div, Pow and the unary maps of ``_EW_UNARY``) whose
    intermediate results are read only inside the group become one ``FusedElementwise`` node: a short
    program for ``mi355x_eltwise_program_f32`` in which every tensor operand is read once and only the final
    result is written -- what the reference leaves to DaCe's map / tasklet fusion after expansion
    (``daceml/transformation/tasklet_fusion.py``). A group is grown backwards from its last node: a producer
    joins when every reader of its result already belongs to the group (so ``g * sigmoid(g)`` keeps ``g`` in
    a register for both readers). An operand is another member's result, a tensor of the result's shape, a
    vector along the last axis, or a scalar constant. When a group does not fit the kernel's limits
    (instructions, registers, operands), members are dropped from its input side until it does. Runs last,
    on whatever the GEMM / Conv epilogue folds and the pattern rewrites left over."""
    from ..onnx.nodes.onnx_op import get_onnx_node

    def fusable(n):
        if _is_op(n, *_EW_BINARY):
            return True
        if _is_op(n, "Gelu"):
            return (n.approximate or "none") == "none"
        return _is_op(n, *_EW_UNARY)

    def io_edges(n):
        ins = [_in_edge(state, n, prm.name) for prm in n.schema.inputs]
        return ins, _out_edge(state, n, n.schema.outputs[0].name)

    def f32_contiguous(desc):
        return desc.dtype.name == "float32" and desc.is_contiguous()

    def readers(acc):
        """Nodes reading the transient behind ``acc`` (one entry per edge), or None when the value is visible
        outside the state's dataflow (not transient, written more than once, or accessed elsewhere)."""
        desc = sdfg.arrays[acc.data]
        if not desc.transient or len(state.in_edges(acc)) != 1:
            return None
        if any(isinstance(n, AccessNode) and n is not acc and n.data == acc.data for n in state.nodes()):
            return None
        return [e.dst for e in state.out_edges(acc)]

    def result_of(n):
        return io_edges(n)[1].dst

    def try_program(members, shape):
        """(program, tensors, vectors, immediates) for ``members`` (operands before their readers), or None when an
        operand cannot be expressed or a limit of the kernel is exceeded."""
        produced = {result_of(m).data: m for m in members}
        uses_left = {}
        for m in members:
            for e in io_edges(m)[0]:
                if e.src.data in produced:
                    uses_left[e.src.data] = uses_left.get(e.src.data, 0) + 1
        tensors, vectors, imms, program, reg_of = [], [], [], [], {}
        free_regs = list(range(8))
        for m in members:
            encoded = []
            for e in io_edges(m)[0]:
                name = e.src.data
                desc = sdfg.arrays[name]
                const = _constant_value(sdfg, name) if not state.in_edges(e.src) else None
                if name in produced:
                    encoded.append((_lib.PROGRAM_REG << 6) | reg_of[name])
                elif const is not None and const.size == 1 and const.dtype == np.float32:
                    v = float(const.reshape(-1)[0])
                    if v not in imms:
                        imms.append(v)
                    encoded.append((_lib.PROGRAM_IMMEDIATE << 6) | imms.index(v))
                elif not f32_contiguous(desc):
                    return None
                elif tuple(desc.shape) == shape:
                    if name not in tensors:
                        tensors.append(name)
                    encoded.append((_lib.PROGRAM_TENSOR << 6) | tensors.index(name))
                elif desc.total_size == shape[-1] and desc.shape and desc.shape[-1] == shape[-1]:
                    if name not in vectors:
                        vectors.append(name)
                    encoded.append((_lib.PROGRAM_VECTOR << 6) | vectors.index(name))
                else:
                    return None     # a broadcast this kernel does not do
            for e in io_edges(m)[0]:     # operands read for the last time give their register back
                name = e.src.data
                if name in produced:
                    uses_left[name] -= 1
                    if uses_left[name] == 0:
                        free_regs.append(reg_of[name])
            if not free_regs:
                return None
            dst = min(free_regs)
            free_regs.remove(dst)
            reg_of[result_of(m).data] = dst
            a = encoded[0]
            b = encoded[1] if len(encoded) > 1 else 0
            if _is_op(m, "Pow") and (b >> 6) == _lib.PROGRAM_IMMEDIATE and imms[b & 63] == 2.0:
                op, b = _lib.OP_MUL, a
            else:
                op = _EW_BINARY.get(m.schema.name, _EW_UNARY.get(m.schema.name))
            program.append(op | (dst << 8) | (a << 16) | (b << 24))
        if len(program) > _lib.PROGRAM_MAX_INSTR or len(tensors) > _lib.PROGRAM_MAX_TENSORS or \
                len(vectors) > _lib.PROGRAM_MAX_VECTORS or len(imms) > _lib.PROGRAM_MAX_IMM:
            return None
        return program, tensors, vectors, imms

    done = set()
    fused = 0
    order = {n: i for i, n in enumerate(state.topological_nodes())}
    for final in sorted((n for n in order if fusable(n)), key=lambda n: -order[n]):
        if final in done or final not in state.nodes():
            continue
        ins, out_e = io_edges(final)
        if out_e is None or not isinstance(out_e.dst, AccessNode) or any(e is None for e in ins):
            continue
        shape = tuple(sdfg.arrays[out_e.dst.data].shape)
        if not shape or not f32_contiguous(sdfg.arrays[out_e.dst.data]):
            continue

        def closure(excluded):
            """Members reachable backwards from ``final`` whose results are read only by members."""
            group = {final}
            changed = True
            while changed:
                changed = False
                for m in list(group):
                    for e in io_edges(m)[0]:
                        prod = _producer(state, e.src)
                        if prod is None or prod.src in group or prod.src in excluded or prod.src in done \
                                or not fusable(prod.src):
                            continue
                        desc = sdfg.arrays[e.src.data]
                        p_ins, p_out = io_edges(prod.src)
                        rd = readers(e.src)
                        if tuple(desc.shape) == shape and f32_contiguous(desc) and rd is not None and \
                                all(r in group for r in rd) and all(pe is not None for pe in p_ins) and p_out is not None:
                            group.add(prod.src)
                            changed = True
            # operands first, depth first from the last node: a valid order that keeps few values alive at once
            ordered, seen = [], set()

            def visit(m):
                if m in seen:
                    return
                seen.add(m)
                for e in io_edges(m)[0]:
                    prod = _producer(state, e.src)
                    if prod is not None and prod.src in group:
                        visit(prod.src)
                ordered.append(m)

            visit(final)
            return ordered

        excluded = set()
        members = closure(excluded)
        built = try_program(members, shape)
        while built is None and len(members) > 2:
            excluded.add(members[0])     # shrink from the input side; the closure drops whatever only fed it
            members = closure(excluded)
            built = try_program(members, shape)
        if built is None or len(members) < 2:
            continue
        program, tensors, vectors, imms = built
        if not (tensors or vectors):
            continue
        # ---- rewrite
        node = get_onnx_node("FusedElementwise")(final.label + "_fused", program=list(program), immediates=list(imms),
                                                 kinds=[_lib.PROGRAM_TENSOR] * len(tensors) + [_lib.PROGRAM_VECTOR] * len(vectors))
        state.add_node(node)
        accesses = {}
        for m in members:
            for e in state.in_edges(m):
                accesses.setdefault(e.src.data, e.src)
        for i, name in enumerate(tensors + vectors):
            node.add_in_connector(f"X__{i}")
            state.add_edge(accesses[name], None, node, f"X__{i}", sdfg.make_array_memlet(name))
        node.add_out_connector("Y")
        state.add_edge(node, "Y", out_e.dst, None, sdfg.make_array_memlet(out_e.dst.data))
        intermediates = [result_of(m) for m in members if m is not final]
        for m in members:
            state.remove_node(m)
            done.add(m)
        for acc in intermediates:
            state.remove_node(acc)
            del sdfg.arrays[acc.data]
        fused += len(members) - 1
    return fused


def _remove_dead_nodes(sdfg: SDFG, state: SDFGState) -> int:
    """Drop nodes whose outputs nobody reads (left behind by the view folds)."""
    removed = 0
    changed = True
    while changed:
        changed = False
        for n in state.nodes():
            if isinstance(n, AccessNode):
                desc = sdfg.arrays.get(n.data)
                if desc is not None and desc.transient and not state.out_edges(n) and state.in_edges(n):
                    prod = state.in_edges(n)[0].src
                    # only pure data-movement nodes are dropped; anything else would be a graph bug
                    if _is_op(prod, "Transpose", "Reshape", "Identity", "Flatten", "Squeeze", "Unsqueeze") and len(state.out_edges(prod)) == 1:
                        state.remove_node(prod)
                        state.remove_node(n)
                        del sdfg.arrays[n.data]
                        removed += 1
                        changed = True
                        break
                elif not state.in_edges(n) and not state.out_edges(n):
                    state.remove_node(n)
                    changed = True
                    break
    return removed


def fuse_onnx_graph(sdfg: SDFG) -> int:
    """Apply every fusion pattern to every state; returns the number of folds."""
    total = 0
    for state in sdfg.nodes():
        total += _fuse_pad_conv(sdfg, state)
        total += _fold_batchnorm_into_conv(sdfg, state)
        total += _fuse_decomposed_layernorm(sdfg, state)
        total += _fuse_decomposed_gelu(sdfg, state)
        total += _fold_into_contractions(sdfg, state)
        total += _fold_operand_scale(sdfg, state)
        total += _fold_views(sdfg, state)
        _remove_dead_nodes(sdfg, state)  # folded Reshape/Transpose chains must not count as readers
        total += _fuse_attention(sdfg, state)
        total += _fuse_shared_input_matmuls(sdfg, state)
        total += _pretranspose_weights(sdfg, state)
        _remove_dead_nodes(sdfg, state)
        total += _fuse_elementwise(sdfg, state)
        _remove_dead_nodes(sdfg, state)
    if total:
        log.info("fused %d patterns in SDFG %s", total, sdfg.name)
    return total

"""Einsum -> one strided batched GEMM: the plan (batch levels, M / N / K and every stride) is evaluated
here by brute force in numpy and compared with numpy's einsum, so the mapping is pinned without a GPU."""
import numpy as np
import pytest

from dace_onnx_amd import sdfg as dace
from dace_onnx_amd.onnx.op_implementations.mi355x_implementations import _einsum_plan


def _desc(a):
    return dace.Array(dace.float32, a.shape, [st // a.itemsize for st in a.strides])


def _run_plan(plan, A, B, out_shape):
    a, b = A.ravel(), B.ravel()
    Y = np.zeros(out_shape)
    y = Y.reshape(-1)
    for b0 in range(plan.batch0):
        for b1 in range(plan.batch1):
            for m in range(plan.M):
                for n in range(plan.N):
                    ia = b0 * plan.a_strides[0] + b1 * plan.a_strides[1] + m * plan.a_strides[2]
                    ib = b0 * plan.b_strides[0] + b1 * plan.b_strides[1] + n * plan.b_strides[3]
                    acc = sum(a[ia + k * plan.a_strides[3]] * b[ib + k * plan.b_strides[2]] for k in range(plan.K))
                    y[b0 * plan.c_strides[0] + b1 * plan.c_strides[1] + m * plan.c_strides[2] + n] = acc
    return Y


@pytest.mark.parametrize("equation, shapes, swapped", [
    ("bij,jk->bik", [(5, 4, 3), (3, 2)], False), ("ik,kj->ij", [(3, 2), (2, 4)], False),
    ("bhqd,bhkd->bhqk", [(2, 3, 6, 4), (2, 3, 5, 4)], False), ("bqhd,bkhd->bhqk", [(2, 6, 3, 4), (2, 5, 3, 4)], False),
    ("bik,jk->bij", [(4, 3, 5), (7, 5)], False), ("ij,bjk->bik", [(6, 5), (3, 5, 8)], False),
    ("bij,bjk->bki", [(3, 6, 5), (3, 5, 8)], True), ("ijk,jkl->il", [(6, 4, 5), (4, 5, 7)], False),
    ("i,j->ij", [(9, ), (12, )], False), ("bi,bi->b", [(6, 10), (6, 10)], False),
    ("abcij,abcjk->abcik", [(2, 2, 2, 3, 4), (2, 2, 2, 4, 5)], False), ("ij,jk->ki", [(3, 4), (4, 5)], True)])
def test_plan_reproduces_numpy_einsum(equation, shapes, swapped):
    rng = np.random.default_rng(3)
    xs = [rng.normal(size=s) for s in shapes]
    expected = np.einsum(equation, *xs)
    found = _einsum_plan(equation, _desc(xs[0]), _desc(xs[1]), _desc(np.zeros(expected.shape)))
    assert found is not None and found[1] == swapped
    A, B = (xs[1], xs[0]) if swapped else (xs[0], xs[1])
    assert np.allclose(_run_plan(found[0], A, B, expected.shape), expected)


def test_bij_jk_folds_the_batch_into_m():
    # the reference's own einsum test (tests/pure_expansions/test_expansions.py:456-473): one 20 x 2 x 3 GEMM
    plan, _ = _einsum_plan("bij ,jk -> bik", _desc(np.zeros((5, 4, 3))), _desc(np.zeros((3, 2))), _desc(np.zeros((5, 4, 2))))
    assert (plan.batch0, plan.batch1, plan.M, plan.N, plan.K) == (1, 1, 20, 2, 3)


@pytest.mark.parametrize("equation, shapes", [("ij,jk->i", [(2, 3), (3, 4)]), ("...ij,jk->...ik", [(2, 2, 3), (3, 4)]),
                                              ("ijk,kjl->il", [(6, 4, 5), (5, 4, 7)]), ("ij,jk", [(2, 3), (3, 4)]),
                                              ("iij,jk->ik", [(3, 3, 2), (2, 4)]), ("ij,jk->ikz", [(2, 3), (3, 4)]),
                                              ("abcdij,abcdjk->acbdik", [(2, 2, 2, 2, 3, 4), (2, 2, 2, 2, 4, 5)])])
def test_what_one_gemm_cannot_do_is_refused(equation, shapes):
    xs = [np.zeros(s) for s in shapes]
    try:
        out_shape = np.einsum(equation, *xs).shape
    except ValueError:
        out_shape = (2, 4, 1)
    assert _einsum_plan(equation, _desc(xs[0]), _desc(xs[1]), _desc(np.zeros(out_shape))) is None

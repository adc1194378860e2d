"""Empty, rank-0 and one-element inputs through the ops added on top of the tables' first pass (match-condition family,
remaining pairwise ops, ReduceBool predicates): no launch on nothing, the reduction's starting value for an empty input,
and the same answers as for ordinary shapes."""
import numpy as np
import pytest

from deeplearning4j_amd.executioner import IndexReduce, Pairwise, ReduceBool, ReduceFloat, ReduceLong, Scalar, TransformBool, TransformSame
from deeplearning4j_amd.ndarray import BOOL, FLOAT32, INT64, NDArray

pytestmark = pytest.mark.gpu


def test_empty_arrays_are_left_alone(ex):
    e = NDArray.from_numpy(np.zeros((0,), np.float32))
    assert ex.exec_transform_bool(TransformBool.MatchConditionBool, e, extra_args=[0.0, 0.0, 10]).to_numpy().shape == (0,)
    assert ex.exec_transform_same(TransformSame.CompareAndSetTransform, e, extra_args=[0.0, 1.0, 0.0, 10]).to_numpy().shape == (0,)
    assert ex.exec_pairwise(Pairwise.CompareAndSet, e, e, extra_args=[0.0, 0.0, 0.0, 10]).to_numpy().shape == (0,)
    assert ex.exec_pairwise(Pairwise.Axpy, e, e, extra_args=[2.0]).to_numpy().shape == (0,)
    assert ex.exec_pairwise(Pairwise.IGamma, e, e).to_numpy().shape == (0,)
    assert ex.exec_scalar(Scalar.CompareAndSet, e, 1.0, extra_args=[0.0, 0.0, 0.0, 10]).to_numpy().shape == (0,)


def test_rank0_and_single_element(ex):
    s = NDArray.from_numpy(np.array(3.0, np.float32))
    assert bool(ex.exec_transform_bool(TransformBool.MatchConditionBool, s, extra_args=[3.0, 0.0, 10]).to_numpy())
    assert float(ex.exec_transform_same(TransformSame.CompareAndSetTransform, s, extra_args=[3.0, 7.0, 0.0, 10]).to_numpy()) == 7.0
    one = NDArray.from_numpy(np.array([3.0], np.float32))
    assert int(ex.exec_index_reduce(IndexReduce.FirstIndex, one, None, extra_args=[3.0, 0.0, 10]).to_numpy()) == 0
    assert int(ex.exec_index_reduce(IndexReduce.LastIndex, one, None, extra_args=[4.0, 0.0, 10]).to_numpy()) == -1
    assert int(ex.exec_reduce_long(ReduceLong.MatchCondition, one, None, extra_args=[3.0, 0.0, 10]).to_numpy()) == 1
    assert float(ex.exec_reduce_float(ReduceFloat.NormP, one, None, extra_args=[3.0]).to_numpy()) == pytest.approx(3.0, rel=1e-6)
    assert bool(ex.exec_reduce_bool(ReduceBool.IsPositive, one).to_numpy()) and not bool(ex.exec_reduce_bool(ReduceBool.IsNegative, one).to_numpy())
    np.testing.assert_allclose(ex.exec_pairwise(Pairwise.IGamma, one, one).to_numpy(), [0.5768099], rtol=1e-5)   # P(3, 3)


def test_reductions_along_a_unit_axis(ex):
    x = np.array([[1.0], [-2.0], [0.0], [np.nan]], np.float32)
    X = NDArray.from_numpy(x)
    assert ex.exec_reduce_long(ReduceLong.MatchCondition, X, [1], extra_args=[0.0, 0.0, 3]).to_numpy().tolist() == [1, 0, 0, 0]     # > 0
    assert ex.exec_index_reduce(IndexReduce.FirstIndex, X, [1], extra_args=[0.0, 0.0, 2]).to_numpy().tolist() == [-1, 0, -1, -1]    # < 0
    assert ex.exec_reduce_bool(ReduceBool.IsNan, X, [1]).to_numpy().tolist() == [False, False, False, True]
    assert ex.exec_reduce_bool(ReduceBool.IsFinite, X, [0]).to_numpy().tolist() == [True]

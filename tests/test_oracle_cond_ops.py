"""Pins the numpy restatements of the match-condition ops against the values the reference's own tests hold
(libnd4j/tests_cpu/layers_tests/NDArrayTests2.cpp:96-103; platform-tests .../nd4j/linalg/indexing/BooleanIndexingTest.java:
208-335): parameter order, which operand is tested, what is returned."""
import numpy as np

from oracle import oracle as O

EPS = 1e-5   # Nd4j.EPS_THRESHOLD, what the Java conditions pass as eps


def test_first_index_reference_vector():
    # ExtraArguments {3.0, 0.0, 10.0}: compare 3, eps 0, mode 10 (==)  ->  index 2
    x = np.array([[1, 2, 3, 4, 5]], np.float64)
    assert O.first_last_index(x, 3.0, 0.0, 10) == 2
    assert O.first_last_index(x, 9.0, 0.0, 10) == -1
    assert O.first_last_index(np.array([1.0, 3, 3, 0]), 3.0, 0.0, 10, last=True) == 2


def test_compare_and_set_transform_reference_vectors():
    x = np.array([1, 2, 0, 4, 5], np.float64)
    assert np.array_equal(O.compare_and_set_transform(x, 0.0, 3.0, EPS, 0), [1, 2, 3, 4, 5])      # testCaSTransform1: equals(0) -> 3
    assert np.array_equal(O.compare_and_set_transform(x, 2.0, 3.0, EPS, 2), [3, 2, 3, 4, 5])      # testCaSTransform2: lessThan(2) -> 3


def test_pairwise_reference_vectors():
    x = np.array([1, 2, 0, 4, 5], np.float64)
    comp = np.array([1, 2, 3, 4, 5], np.float64)
    # testCaSPairwiseTransform1: CompareAndSet(x, comp, lessThan(5)) -> comp (the second operand is tested: 1,2,3,4 < 5 taken, 5 kept)
    assert np.array_equal(O.compare_and_set(x, comp, 5.0, EPS, 2), comp)
    # testCaRPairwiseTransform1: CompareAndReplace(x, comp, lessThan(1)) -> comp (only x = 0 is replaced)
    assert np.array_equal(O.compare_and_replace(x, comp, 1.0, EPS, 2), comp)
    y = np.array([2, 4, 3, 0, 5], np.float64)
    # testCaSPairwiseTransform2: CompareAndSet(x, y, epsNotEquals(0)) -> [2,4,3,4,5] (y = 0 is not taken)
    assert np.array_equal(O.compare_and_set(x, y, 0.0, EPS, 1), [2, 4, 3, 4, 5])
    y2 = np.array([2, 4, 3, 4, 5], np.float64)
    assert np.array_equal(O.compare_and_replace(x, y2, 0.0, EPS, 1), [2, 4, 0, 4, 5])             # testCaRPairwiseTransform2
    assert np.array_equal(O.compare_and_replace(x, y2, 4.0, EPS, 2), [2, 4, 3, 4, 5])             # testCaSPairwiseTransform3
    assert np.array_equal(O.compare_and_replace(x, y2, 2.0, EPS, 2), [2, 2, 3, 4, 5])             # testCaRPairwiseTransform3


def test_match_count_reference_vectors():
    a = np.arange(10, dtype=np.float64)
    assert O.match_count(a, 5.0, EPS, 2) == 5                                                     # testMatchConditionAllDimensions1
    b = a.copy(); b[4] = np.nan
    assert O.match_count(b, 0.0, EPS, 9) == 1                                                     # ...2: isNan
    c = a.copy(); c[4] = -np.inf
    assert O.match_count(c, 0.0, EPS, 8) == 1                                                     # ...3: isInfinite
    m = np.ones((3, 10)); m[2] = 0
    assert np.array_equal(O.match_count(m, 0.0, EPS, 0, dims=[1]) == 10, [False, False, True])    # testMatchConditionAlongDimension1


def test_norm_p_and_equals_with_eps_closed_forms():
    x = np.array([[3.0, -4.0], [1.0, 1.0]])
    np.testing.assert_allclose(O.norm_p(x, 2.0, dims=[1]), [5.0, np.sqrt(2)])
    np.testing.assert_allclose(O.norm_p(x, 1.0), 9.0)
    np.testing.assert_allclose(O.norm_p(x, 3.0, dims=[0]), [(27 + 1) ** (1 / 3), (64 + 1) ** (1 / 3)])
    assert O.equals_with_eps(x, x + 1e-7, 1e-5) == 1.0 and O.equals_with_eps(x, x + 1e-3, 1e-5) == 0.0

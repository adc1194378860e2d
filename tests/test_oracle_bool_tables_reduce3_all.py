"""The oracle's restatement of the bool tables (pairwise / scalar / broadcast ops with a BOOL result), pinned by the
reference's own test vectors and by facts that do not come from the restatement: numpy's logical routines, the
boundary values of the tolerance, truth tables written out by hand."""
import numpy as np
import pytest

from oracle import oracle as O

EQ, GT, LT, EPS, GE, NE, AND, OR, XOR, NOT, LE = 0, 1, 2, 3, 4, 6, 7, 8, 9, 10, 11


def test_reference_vectors_pairwise_equal_to():
    # MultiDataTypeTests.cpp:1095-1124 (ndarray_applyPairwiseTransform_test2): arrays of one length and different shapes
    # are walked by linear index
    x1, x2 = np.array([1, 1, 2, 3, 4, 5], np.int32), np.array([1, 0, 2, 0, 4, 0], np.int32)
    assert O.bool_table(EQ, x1, x2).tolist() == [1, 0, 1, 0, 1, 0]
    x3, x4 = np.array([0.5, 1.5, 2.5, 3, 4.5, 0]), np.array([0.5, 1., 2.5, 3, 4., 0])
    assert O.bool_table(EQ, x3, x4).tolist() == [1, 0, 1, 1, 0, 1]
    x5, x6 = np.array([0, 1, 0, 1, 0, 1], bool), np.array([1, 1, 1, 0, 1, 0], bool)
    assert O.bool_table(EQ, x5, x6).tolist() == [0, 1, 0, 0, 0, 0]


def test_reference_vectors_broadcast_and_scalar():
    # MultiDataTypeTests.cpp:1150-1172 (ndarray_applyBroadcast_test2): y along dimension 0
    x1, x2 = np.array([[10, 20, 30], [40, 50, 60]], np.int32), np.array([10, 60], np.int32)
    assert O.bool_table(EQ, x1, O.operand_along(x2, x1.shape, [0])).reshape(-1).tolist() == [1, 0, 0, 0, 0, 1]
    x4, x5 = np.array([[0, 0, 0], [0, 0, 1]], bool), np.array([0, 1], bool)
    assert O.bool_table(EQ, x4, O.operand_along(x5, x4.shape, [0])).reshape(-1).tolist() == [1, 1, 1, 0, 0, 1]
    # MultiDataTypeTests.cpp:1290-1311 (ndarray_applyScalar_test2)
    for x, s, want in ((np.array([0, 1, 2, 3], np.int64), 1, [0, 1, 0, 0]), (np.array([0, 1.5, 2.5, 3.5], np.float32), 1.5, [0, 1, 0, 0]),
                       (np.array([0, 1, 1, 0], bool), True, [0, 1, 1, 0])):
        assert O.bool_table(EQ, x, np.full(x.shape, s, x.dtype)).tolist() == want
    # NativeOpsTests.cpp:144-167 (ExecBroadcast_2): x = 1..25 as [5, 5], y = 2, 4, .., 10 along dimension 0
    x = np.arange(1, 26, dtype=np.float32).reshape(5, 5)
    z = O.bool_table(EQ, x, O.operand_along(np.arange(2, 11, 2, dtype=np.float32).reshape(5, 1), x.shape, [0])).reshape(-1)
    assert z[1] and not z[0]
    # NativeOpsTests.cpp:186-206 (ExecPairwise_2): And of all-true with a single true
    y = np.zeros(25, bool); y[5] = True
    z = O.bool_table(AND, np.ones(25, bool), y)
    assert z[5] and not z[4]
    # NativeOpsTests.cpp:803-832 (ScalarTadTest_2): And with one scalar for the whole array (dimensions 0, 1)
    xb = np.zeros((5, 5), bool); xb.reshape(-1)[[5, 15]] = True
    z = O.bool_table(AND, xb, O.scalars_along(np.array([True]), xb.shape, [0, 1])).reshape(-1)
    assert z[5] and z[15] and z.sum() == 2


def test_operand_shapes_follow_the_loops():
    # broadcasting: y's dims line up with `dims` of x, in order; unit dims of y and of x are skipped
    x_shape = (1, 3, 2, 4, 4)                                   # DeclarableOpsTests9.cpp:811-821 (test_broadcast_bool_1)
    y = np.arange(32.0).reshape(1, 2, 4, 4)
    full = O.operand_along(y, x_shape, [0, 2, 3, 4])
    assert full.shape == x_shape
    for i in range(3):
        assert np.array_equal(full[0, i], y[0])
    # one scalar per sub-array: numbered in c order over the other dims
    s = np.arange(6.0)
    full = O.scalars_along(s, (2, 5, 3), [1])
    for a in range(2):
        for b in range(3):
            assert np.all(full[a, :, b] == s[a * 3 + b])
    # ScalarTadTest_1 (NativeOpsTests.cpp:762-793): one scalar, dimensions 0 and 1
    assert np.all(O.scalars_along(np.array([10.0]), (5, 5), [0, 1]) == 10.0)


@pytest.mark.parametrize("dtype", [np.float64, np.float32, np.float16, np.int32, np.int64])
def test_comparisons_are_numpys(dtype):
    rng = np.random.default_rng(3)
    x, y = rng.integers(-3, 4, 500).astype(dtype), rng.integers(-3, 4, 500).astype(dtype)
    for op, fn in ((EQ, np.equal), (GT, np.greater), (LT, np.less), (GE, np.greater_equal), (NE, np.not_equal), (LE, np.less_equal), (NOT, np.not_equal)):
        assert np.array_equal(O.bool_table(op, x, y), fn(x, y)), op


def test_comparisons_with_nan_are_false_except_not_equal():
    x, y = np.array([np.nan, 1.0, np.nan], np.float32), np.array([1.0, np.nan, np.nan], np.float32)
    for op in (EQ, GT, LT, GE, LE):
        assert not O.bool_table(op, x, y).any()
    assert O.bool_table(NE, x, y).all() and O.bool_table(NOT, x, y).all()


def test_logic_truth_tables():
    a, b = np.array([0, 0, 1, 1], bool), np.array([0, 1, 0, 1], bool)
    assert O.bool_table(AND, a, b).tolist() == [0, 0, 0, 1]
    assert O.bool_table(OR, a, b).tolist() == [0, 1, 1, 1]
    assert O.bool_table(XOR, a, b).tolist() == [0, 1, 1, 0]
    # numbers count as true when not zero (NaN included), and the three agree with numpy's logical routines
    x, y = np.array([0.0, -2.0, np.nan, 0.0, 3.0], np.float32), np.array([0.0, 0.0, 0.0, 5.0, np.nan], np.float32)
    assert np.array_equal(O.bool_table(AND, x, y), np.logical_and(x, y))
    assert np.array_equal(O.bool_table(OR, x, y), np.logical_or(x, y))
    assert np.array_equal(O.bool_table(XOR, x, y), np.logical_xor(x, y))
    # with a parameter c the tests are "differs from c": And -> neither is c, Or -> not both are c, Xor -> exactly one is c
    x, y = np.array([7, 7, 1, 2], np.int32), np.array([7, 3, 7, 5], np.int32)
    assert O.bool_table(AND, x, y, [7]).tolist() == [0, 0, 0, 1]
    assert O.bool_table(OR, x, y, [7]).tolist() == [0, 1, 1, 1]
    assert O.bool_table(XOR, x, y, [7]).tolist() == [0, 1, 1, 0]
    # c = 0 reproduces the parameterless tables
    for op in (AND, OR, XOR):
        assert np.array_equal(O.bool_table(op, x - 7, y - 7, [0]), O.bool_table(op, x - 7, y - 7))


def test_epsilon_boundaries():
    # the default tolerance is 1e-5 as the type holds it: float32(1e-5) lies above 1e-5, so a float32 difference of exactly
    # float32(1e-5) passes and the next float up does not; the integer types hold 0: only equal values pass
    t = np.float32(1e-5)
    x = np.zeros(3, np.float32)
    y = np.array([t, np.nextafter(t, np.float32(1)), -t], np.float32)
    assert O.bool_table(EPS, x, y).tolist() == [1, 0, 1]
    assert O.bool_table(EPS, np.array([1, 2, 3], np.int32), np.array([1, 3, 2], np.int32)).tolist() == [1, 0, 0]
    # a given tolerance widens the default one, it never narrows it (the default test still applies)
    x, y = np.zeros(4), np.array([0.5, 0.25, 1e-6, 1e-5 * 1.5])
    assert O.bool_table(EPS, x, y, [0.25]).tolist() == [0, 1, 1, 1]
    assert O.bool_table(EPS, x, y, [1e-9]).tolist() == [0, 0, 1, 0]
    # half and bfloat16 hold 1e-5 as the same number, 168 * 2^-24
    assert float(np.float16(1e-5)) == 168.0 / 2 ** 24
    assert float(O.bf16_to_f32(O.f32_to_bf16(np.array([1e-5], np.float32)))[0]) == 168.0 / 2 ** 24
    h = np.float16(168.0 / 2 ** 24)
    assert O.bool_table(EPS, np.zeros(2, np.float16), np.array([h, np.nextafter(h, np.float16(1))], np.float16)).tolist() == [1, 0]
    # differences are rounded to the storage type first: 1 + 2^-9 is not a bfloat16, so the inputs below are 1 and 1.0078125
    xb = O.bf16_to_f32(O.f32_to_bf16(np.array([1.0, 1.0], np.float32)))
    yb = O.bf16_to_f32(O.f32_to_bf16(np.array([1.0, 1.0078125], np.float32)))
    assert O.bool_table(EPS, xb, yb, None, bf16=True).tolist() == [1, 0]
    assert O.bool_table(EPS, xb, yb, [0.0078125], bf16=True).tolist() == [1, 1]


def test_reduce3_all_reference_vectors():
    # NDArrayTests.cpp:1455-1470 (applyAllReduce3EuclideanDistance): rows of x against rows of y
    x, y = np.array([[1, 2, 3], [4, 5, 6]], np.float32), np.full((2, 3), 2, np.float32)
    np.testing.assert_allclose(O.reduce3_all(1, x, y, [1]), [[1.414214, 1.414214], [5.385165, 5.385165]], rtol=1e-6)
    # NDArrayTests2.cpp:186-209 (Test_AllReduce3_1 / _2)
    a, b = np.array([[1, 2, 3], [1, 2, 3]], np.float64), np.array([[2, 3, 4], [2, 3, 4]], np.float64)
    np.testing.assert_allclose(O.reduce3_all(1, a, b, [1]), np.full((2, 2), 1.73205), rtol=1e-5)
    c = np.array([[1, 2, 3], [2, 3, 4]], np.float64)
    np.testing.assert_allclose(O.reduce3_all(1, c, c, [1]), [[0, 1.73205], [1.73205, 0]], rtol=1e-5)
    # MultiDataTypeTests.cpp:1629-1644 (applyAllReduce3_test1): Dot over the columns (dimension 0), operands of different widths
    x4, x3 = np.array([[1, 2], [3, 4]], np.float64), np.full((2, 3), 1.5)
    assert np.array_equal(O.reduce3_all(3, x4, x3, [0]), [[6, 6, 6], [9, 9, 9]])
    x1, x2 = np.array([[1, 2], [3, 4]], np.float64), np.array([[-1, 1, -1], [1, -1, 1]], np.float64)
    assert np.array_equal(O.reduce3_all(3, x1, x2, [0]), [[2, -2, 2], [2, -2, 2]])


def test_reduce3_all_dot_is_a_matrix_product():
    rng = np.random.default_rng(9)
    x, y = rng.integers(-4, 5, (5, 7)).astype(np.float64), rng.integers(-4, 5, (6, 7)).astype(np.float64)
    assert np.array_equal(O.reduce3_all(3, x, y, [1]), x @ y.T)
    # sub-arrays of rank 2, the other dims numbered in c order
    x3, y3 = rng.integers(-4, 5, (2, 4, 3, 5)).astype(np.float64), rng.integers(-4, 5, (3, 4, 2, 5)).astype(np.float64)
    want = np.einsum("aibk,cidk->abcd", x3, y3).reshape(6, 6)
    assert np.array_equal(O.reduce3_all(3, x3, y3, [1, 3]), want)

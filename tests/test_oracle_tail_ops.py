"""Pins of the oracle's long-tail transform / pairwise / scalar / broadcast restatements (CPU only).

The reference holds no vectors for these ops, so each is checked against what the mathematics fixes:
library routines (numpy, scipy.special, math), identities, and -- for every *Derivative op -- the central
difference of the oracle's own primal op in float64, which a wrong sign, factor or constant fails.
"""
import math

import numpy as np
import pytest
import scipy.special as sp

from oracle import oracle as O

S = dict(TanhD=4, SigmoidD=6, SoftSignD=7, TanD=8, SELUD=9, RationalTanhD=11, RectifiedTanhD=12, SwishD=13, ACoshD=14,
         ASinhD=15, SinhD=16, LogSigmoidD=17, SpecialD=18, CubeD=21, Cosine=22, Exp=23, Log=24, Sigmoid=26, Sin=27,
         SoftPlus=28, Tanh=29, ACos=30, ASin=31, ATan=32, HardTanh=33, SoftSign=34, HardSigmoid=36, RationalTanh=37,
         RectifiedTanh=38, Sinh=39, Cosh=40, Tan=41, SELU=42, Swish=43, Log1p=44, ACosh=46, ASinh=47, Rint=48,
         LogSigmoid=49, Erfc=50, Expm1=51, ATanh=52, GELU=53, GELUD=54, PGELU=55, PGELUD=56, Mish=57, MishD=58)


def strict(op, x):
    x = np.ascontiguousarray(x)
    return O.transform_strict(op, x, np.zeros_like(x))


GRID = np.linspace(-4.0, 4.0, 161)

PRIMAL = [
    (S["ACos"], np.linspace(-1, 1, 81), np.arccos),
    (S["ASin"], np.linspace(-1, 1, 81), np.arcsin),
    (S["ATan"], GRID, np.arctan),
    (S["HardTanh"], GRID, lambda x: np.clip(x, -1, 1)),
    (S["SoftSign"], GRID, lambda x: x / (1 + np.abs(x))),
    (S["HardSigmoid"], GRID, lambda x: np.clip(np.float64(np.float32(0.2)) * x + 0.5, 0, 1)),   # slope is the float constant 0.2f
    (S["RectifiedTanh"], GRID, lambda x: np.maximum(0, np.tanh(x))),
    (S["Sinh"], GRID, np.sinh),
    (S["Cosh"], GRID, np.cosh),
    (S["Tan"], np.linspace(-1.4, 1.4, 57), np.tan),
    (S["Log1p"], np.linspace(-0.9, 5, 60), np.log1p),
    (S["ACosh"], np.linspace(1.0, 9, 81), np.arccosh),
    (S["ASinh"], GRID, np.arcsinh),
    (S["Rint"], np.linspace(-3.5, 3.5, 29), np.rint),                 # 0.25 steps: halves go to even
    (S["LogSigmoid"], GRID, lambda x: -np.logaddexp(0, -x)),          # log sigma(x) = -log(1 + e^-x)
    (S["Erfc"], GRID, sp.erfc),
    (S["Expm1"], GRID, np.expm1),
    (S["ATanh"], np.linspace(-0.95, 0.95, 77), np.arctanh),
    (S["Mish"], GRID, lambda x: x * np.tanh(np.logaddexp(0, x))),
]


@pytest.mark.parametrize("op,x,fn", PRIMAL, ids=[str(p[0]) for p in PRIMAL])
def test_strict_primal_ops_match_library_routines(op, x, fn):
    want = fn(x)
    np.testing.assert_allclose(strict(op, x.astype(np.float64)), want, rtol=1e-12, atol=1e-13)
    got32 = strict(op, x.astype(np.float32)).astype(np.float64)
    w32 = fn(x.astype(np.float32).astype(np.float64))
    np.testing.assert_allclose(got32, w32, rtol=2e-6, atol=3e-7)


def test_selu_constants_and_shape():
    lam, alpha = 1.0507009873554805, 1.6732632423543772      # Klambauer et al. 2017, eq. (fixed point 0, 1)
    x = np.array([-50.0, -1.0, 0.0, 1.0, 3.0])
    got = strict(S["SELU"], x)
    assert got[3] == pytest.approx(lam, rel=1e-15) and got[4] == pytest.approx(3 * lam, rel=1e-15)
    assert got[0] == pytest.approx(-lam * alpha, rel=1e-12)   # saturation value -1.7581
    assert got[1] == pytest.approx(lam * alpha * (math.exp(-1) - 1), rel=1e-14)
    assert got[2] == 0.0


def test_rational_tanh_tracks_scaled_tanh():
    x = np.linspace(-6, 6, 241)
    got = strict(S["RationalTanh"], x)
    assert np.max(np.abs(got - 1.7159 * np.tanh(2 * x / 3))) < 0.03        # the approximation it is built to be
    np.testing.assert_allclose(got, -got[::-1], rtol=0, atol=1e-14)         # odd
    assert np.all(np.diff(got) > 0)                                         # increasing


DERIV = [  # (derivative op, primal op, grid)
    (S["TanhD"], S["Tanh"], GRID), (S["SigmoidD"], S["Sigmoid"], GRID), (S["SoftSignD"], S["SoftSign"], GRID[GRID != 0]),
    (S["TanD"], S["Tan"], np.linspace(-1.3, 1.3, 53)), (S["SELUD"], S["SELU"], GRID[GRID != 0]),
    (S["RationalTanhD"], S["RationalTanh"], GRID[GRID != 0]), (S["RectifiedTanhD"], S["RectifiedTanh"], GRID[GRID != 0]),
    (S["SwishD"], S["Swish"], GRID), (S["ACoshD"], S["ACosh"], np.linspace(1.2, 9, 40)), (S["ASinhD"], S["ASinh"], GRID),
    (S["SinhD"], S["Sinh"], GRID), (S["LogSigmoidD"], S["LogSigmoid"], GRID), (S["GELUD"], S["GELU"], GRID),
    (S["MishD"], S["Mish"], GRID),
]


@pytest.mark.parametrize("dop,pop,x", DERIV, ids=[str(d[0]) for d in DERIV])
def test_derivative_ops_match_central_differences_of_their_primal(dop, pop, x):
    h = 1e-6
    x = np.ascontiguousarray(x, dtype=np.float64)
    num = (strict(pop, x + h) - strict(pop, x - h)) / (2 * h)
    np.testing.assert_allclose(strict(dop, x), num, rtol=2e-7, atol=2e-8)
    got32 = strict(dop, x.astype(np.float32)).astype(np.float64)
    np.testing.assert_allclose(got32, num, rtol=1e-4, atol=1e-5)


def test_precise_gelu_derivative_properties():
    # The reference writes this op as 0.5 + (0.398942 x + (0.0535161 x)^3) sech^2(u) + 0.5 tanh(u) with
    # u = 0.797885 x + (0.0356774 x)^3: the cubes wrap the scaled argument, so away from zero it is neither the derivative
    # of the textbook tanh-GELU nor of the reference's own PreciseGELU (values there: parity unpinned).  What holds for any
    # function of this form: f'(x) + f'(-x) = 1, and the textbook derivative near zero where the cubic terms vanish.
    x = GRID
    got = strict(S["PGELUD"], x)
    np.testing.assert_allclose(got + got[::-1], 1.0, rtol=0, atol=1e-15)
    small = np.linspace(-0.02, 0.02, 21)
    f = lambda v: 0.5 * v * (1 + np.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3)))
    h = 1e-6
    num = (f(small + h) - f(small - h)) / (2 * h)
    np.testing.assert_allclose(strict(S["PGELUD"], small), num, rtol=0, atol=2e-6)


def test_polynomial_derivatives():
    x = GRID
    np.testing.assert_array_equal(strict(S["SpecialD"], x), x * (1 - x))
    np.testing.assert_array_equal(strict(S["CubeD"], x), 3 * x * x)


def test_transform_same_ops():
    x = np.linspace(-3.75, 3.75, 61)          # 0.125 steps: exact halves included
    same = lambda op: O.transform_same(op, x, np.zeros_like(x))
    np.testing.assert_array_equal(same(2), np.ones_like(x))
    np.testing.assert_array_equal(same(4), np.sign(x) * np.floor(np.abs(x) + 0.5))     # halves away from zero
    assert same(4)[np.where(x == 2.5)[0][0]] == 3.0 and same(4)[np.where(x == -2.5)[0][0]] == -3.0
    np.testing.assert_array_equal(same(5), x * (1 - x))
    np.testing.assert_array_equal(same(17), np.ceil(x))
    np.testing.assert_array_equal(same(18), np.floor(x))
    np.testing.assert_array_equal(same(0), np.abs(x))
    np.testing.assert_array_equal(same(6), x ** 3)
    # Sign: the reference's macro takes the sign expression as its CONDITION (ops.h:217-219 through
    # op_macros_unary.h:109-113), i.e. ((d1 > 0) - (d1 < 0)) ? 1 : -1.  Evaluated by hand: -3 -> (0 - 1) = -1, non-zero -> 1;
    # 0 -> 0 -> -1; 2 -> 1 -> 1; NaN -> (0 - 0) = 0 -> -1
    np.testing.assert_array_equal(O.transform_same(1, np.array([-3.0, 0.0, 2.0, np.nan, -0.0]), np.zeros(5)), [1.0, -1.0, 1.0, -1.0, -1.0])
    np.testing.assert_array_equal(O.transform_same(1, np.array([-3.0, 0.0, 2.0], np.float32), np.zeros(3, np.float32)), [1.0, -1.0, 1.0])


def test_strict_ops_whose_macros_return_the_input():
    # HardTanhDerivative (5) and HardSigmoidDerivative (10): (CONDITION) ? d1 : d1 -- the input whatever the condition says;
    # StabilizeFP16 (20): x <= 0 ? 2^-14 : x (ops.h:381-384; 2^-14 = 6.103515625e-05 is float16's smallest normal number,
    # which is what static_cast<float16>(6.1035e-05) rounds to: the neighbouring subnormal 1023 * 2^-24 is 5.96e-8 further away)
    x = np.array([-3.0, -1.0, -0.5, 0.0, 0.5, 1.0, 2.5, 2.6, 7.0])
    for dt in (np.float32, np.float64):
        xt = x.astype(dt)
        np.testing.assert_array_equal(O.transform_strict(5, xt, np.zeros_like(xt)), xt)
        np.testing.assert_array_equal(O.transform_strict(10, xt, np.zeros_like(xt)), xt)
        np.testing.assert_array_equal(O.transform_strict(20, xt, np.zeros_like(xt)), np.where(x <= 0, 2.0 ** -14, x).astype(dt))
    assert np.float16(6.1035e-05) == np.float16(2.0 ** -14)


def test_transform_float_takes_integer_and_bool_inputs():
    # NativeOpExecutioner_transform.cpp:35-37: any common type into any float type; sd_sqrt<X, Z> converts to Z first
    for xdt in (np.int32, np.int64):
        x = np.array([0, 1, 4, 9, 16, 2, 1000003], xdt)
        np.testing.assert_array_equal(O.transform_float(1, x, np.zeros(x.shape, np.float32)), np.sqrt(x.astype(np.float32)))
        np.testing.assert_array_equal(O.transform_float(1, x, np.zeros(x.shape, np.float64)), np.sqrt(x.astype(np.float64)))
    b = np.array([True, False, True])
    np.testing.assert_array_equal(O.transform_float(1, b, np.zeros(3, np.float32)), [1.0, 0.0, 1.0])
    h = O.transform_float(3, np.array([4, 16], np.int32), np.zeros(2, np.float16))
    np.testing.assert_array_equal(h, np.array([0.5, 0.25], np.float16))


def test_reduce_float_of_other_input_types():
    # MultiDataTypeTests.cpp:246-256 (ndarray_reduceAlongDimension_test2): Mean of INT32 {0, 1, 2, 3} into FLOAT32
    x = np.array([[0, 1], [2, 3]], np.int32)
    assert O.reduce_float(0, x, np.zeros((), np.float32)) == np.float32(1.5)
    np.testing.assert_array_equal(O.reduce_float(0, x, np.zeros(2, np.float32), [1]), np.array([0.5, 2.5], np.float32))
    # the accumulator follows Z (op_macros_reduce.h:778-782): fp32 values whose fp32 running sum loses the small terms
    # are summed exactly when Z is DOUBLE
    v = np.array([1e8, 1.0, 1.0, 1.0, 1.0, -1e8], np.float32)
    assert O.reduce_float(0, v, np.zeros((), np.float64)) == 4.0 / 6.0
    assert O.reduce_float(0, v, np.zeros((), np.float32)) == np.float32(0.0)      # 1e8 + 1 == 1e8 in fp32
    rng = np.random.default_rng(5)
    for xdt in (np.int64, np.float16, np.float64, np.bool_):
        a = rng.integers(0, 2, (5, 7)).astype(xdt) if xdt == np.bool_ else (rng.uniform(-4, 4, (5, 7)) * 3).astype(xdt)
        a64 = a.astype(np.float64)
        for op, want in ((0, a64.mean(1)), (1, np.abs(a64).mean(1)), (2, np.abs(a64).sum(1)), (3, np.sqrt((a64 ** 2).sum(1))),
                         (4, np.abs(a64).max(1)), (7, (a64 ** 2).sum(1))):
            np.testing.assert_allclose(O.reduce_float(op, a, np.zeros(5, np.float32), [1]), want, rtol=2e-6, atol=1e-6)
            np.testing.assert_allclose(O.reduce_float(op, a, np.zeros(5, np.float64), [1]), want, rtol=1e-12, atol=1e-12)


def test_reductions_of_empty_arrays():
    # LegacyOpsTests.cpp:616-658 (test_legacy_reduce_empty_1/2/3): Sum of [2, 0, 3] along 1 -> zeros, Min -> +inf, Max -> -inf;
    # DeclarableOpsTests14.cpp:230-265: reduce_min of a float [1, 0] -> infOrMax<float>, reduce_sum -> 0, reduce_mean -> NaN
    f32 = np.dtype(np.float32)
    assert O.reduce_of_empty("same", 0, f32, f32) == 0
    assert O.reduce_of_empty("same", 2, f32, f32) == np.inf and O.reduce_of_empty("same", 1, f32, f32) == -np.inf
    assert np.isnan(O.reduce_of_empty("float", 0, f32, f32))
    # DeclarableOpsTests14.cpp:306-317 argmax of an empty array gives an empty result; the loop's own fill is index 0
    assert O.reduce_of_empty("index", 0, f32, np.dtype(np.int64)) == 0 and O.reduce_of_empty("index", 4, f32, np.dtype(np.int64)) == -1
    # infOrMax / nanOrZero are specialised for float and double only (array/DataTypeUtils.h:600-636)
    assert O.reduce_of_empty("same", 1, "float16", "float16") == -65504.0
    assert O.reduce_of_empty("same", 2, "bfloat16", "bfloat16") == float(np.float32(2.0 ** 127 * (2 - 2.0 ** -7)))
    assert O.reduce_of_empty("same", 1, np.dtype(np.int32), np.dtype(np.int32)) == -(2 ** 31 - 1)
    assert O.reduce_of_empty("float", 0, np.dtype(np.int32), "float16") == 0.0
    assert O.reduce_of_empty("same", 3, f32, f32) == 1 and O.reduce_of_empty("bool", 1, f32, np.dtype(bool)) == 1
    assert O.reduce_of_empty("same", 5, f32, f32) is None


def test_matmul_of_integer_arrays():
    # the reference's loop in the arrays' own type (MmulHelper.cpp:35-110) against Python's exact integers reduced modulo 2^bits
    rng = np.random.default_rng(11)
    for dt, bits in ((np.int32, 32), (np.int64, 64)):
        a = rng.integers(-2 ** (bits - 2), 2 ** (bits - 2), (3, 5)).astype(dt)
        b = rng.integers(-2 ** (bits - 2), 2 ** (bits - 2), (5, 4)).astype(dt)
        c = rng.integers(-100, 100, (3, 4)).astype(dt)
        def wrap(v):
            v %= 2 ** bits
            return v - 2 ** bits if v >= 2 ** (bits - 1) else v
        for alpha, beta in ((1.0, 0.0), (3.0, 2.0), (2.9, 0.0)):
            want = np.array([[wrap(int(alpha) * sum(int(a[i, k]) * int(b[k, j]) for k in range(5)) + (int(beta) * int(c[i, j]) if beta else 0))
                              for j in range(4)] for i in range(3)], dtype=dt)
            np.testing.assert_array_equal(O.matmul_int(a, b, c, alpha, beta), want)
    # DeclarableOpsTests-style small case: exact products
    np.testing.assert_array_equal(O.matmul_int(np.array([[1, 2], [3, 4]], np.int32), np.array([[5, 6], [7, 8]], np.int32)), [[19, 22], [43, 50]])


def _c_int_div(a, b):
    return np.trunc(a.astype(np.int64).astype(np.float64) / b.astype(np.int64)).astype(np.float64)


def _c_int_mod(a, b):
    return np.fmod(a.astype(np.int64), b.astype(np.int64)).astype(np.float64)


A = np.array([-7.5, -5.5, -3.0, -1.25, 0.0, 0.5, 2.0, 3.75, 5.5, 7.0, 9.25, -9.0])
B = np.array([2.0, -2.0, 4.0, 3.5, 1.5, -1.5, 3.0, -1.25, 2.5, 3.0, -4.0, 2.0])      # (int)b is never zero

BINARY = {  # pairwise opNum -> independent routine
    4: lambda a, b: np.power(np.abs(a) + 0.5, b),
    14: lambda a, b: np.array([math.remainder(u, v) for u, v in zip(a, b)]),
    15: np.fmod,
    16: np.arctan2,
    17: _c_int_div,
    18: lambda a, b: np.floor(a / b),
    19: np.mod,                                  # sign follows the divisor
    21: lambda a, b: _c_int_mod(b, np.where(a.astype(np.int64) == 0, 1, a)),
    22: lambda a, b: a / b,
    23: np.mod,                                  # a - floor(a/b) b
    27: lambda a, b: (a.astype(np.int64) | b.astype(np.int64)).astype(np.float64),
    28: lambda a, b: (a.astype(np.int64) ^ b.astype(np.int64)).astype(np.float64),
    30: lambda a, b: (a.astype(np.int64) & b.astype(np.int64)).astype(np.float64),
    29: lambda a, b: (~((a.astype(np.int64) != 0) & (b.astype(np.int64) != 0))).astype(np.float64),
    34: lambda a, b: np.where(np.abs(a) > np.abs(b), a, b),
    35: lambda a, b: np.where(np.abs(a) < np.abs(b), a, b),
    36: _c_int_mod,
    38: lambda a, b: a / b,
}


@pytest.mark.parametrize("op", sorted(BINARY))
def test_pairwise_tail_ops(op):
    a, b = A.copy(), B.copy()
    if op == 4:
        a = np.abs(a) + 0.5
    if op == 21:
        a = np.where(a.astype(np.int64) == 0, 1.0, a)
    want = BINARY[op](A if op == 4 else a, b)
    got = O.pairwise(op, a, b, np.zeros_like(a))
    np.testing.assert_allclose(got, want, rtol=1e-14, atol=0)
    got32 = O.pairwise(op, a.astype(np.float32), b.astype(np.float32), np.zeros(a.shape, np.float32))
    np.testing.assert_allclose(got32, want, rtol=1e-6, atol=1e-7)


def test_pairwise_zero_divisors_and_nans():
    a = np.array([1.0, -2.0, np.nan, 0.0])
    b = np.array([0.0, 0.0, 5.0, 0.0])
    np.testing.assert_array_equal(O.pairwise(22, a, b, np.zeros(4)), [0, 0, np.nan, 0])     # SafeDivide
    np.testing.assert_array_equal(O.pairwise(38, a, b, np.zeros(4)), [0, 0, np.nan, 0])     # DivideNoNan
    np.testing.assert_array_equal(O.pairwise(37, a, b, np.zeros(4)), [1, -2, 5, 0])         # ReplaceNans


def test_scalar_table_numbers_each_function():
    x = np.array([-7.5, -2.0, -0.5, 0.0, 0.5, 2.0, 7.0])
    sc = lambda op, v, xx=x: O.scalar(op, xx, v, np.zeros_like(xx))
    np.testing.assert_allclose(sc(7, 1.5), np.where(x >= 0, x, 1.5 * np.expm1(x)), rtol=1e-14)            # ELU
    np.testing.assert_allclose(sc(8, 1.5), np.where(x >= 0, 1, 1.5 * np.exp(x)), rtol=1e-14)              # ELUDerivative
    np.testing.assert_array_equal(sc(15, 3.0), np.mod(x, 3.0))                                            # Mod
    np.testing.assert_array_equal(sc(16, 7.0, np.array([2.0, 3.0, -4.0])), [1, 1, 3])                     # ReverseMod: 7 % (int)x
    np.testing.assert_array_equal(sc(17, 3.0), [math.remainder(v, 3.0) for v in x])                       # Remainder
    np.testing.assert_array_equal(sc(18, 3.0), np.fmod(x, 3.0))                                           # FMod
    np.testing.assert_array_equal(sc(19, 2.0), np.trunc(np.trunc(x) / 2))                                 # TruncateDiv
    np.testing.assert_array_equal(sc(20, 2.0), np.floor(x / 2))                                           # FloorDiv
    np.testing.assert_array_equal(sc(21, -3.0), np.mod(x, -3.0))                                          # FloorMod
    np.testing.assert_array_equal(sc(22, 1.0), (x - 1) ** 2)
    np.testing.assert_array_equal(sc(44, 1.0), (1 - x) ** 2)
    np.testing.assert_array_equal(sc(24, 1.0), np.where(np.abs(x) > 1, x, 1.0))                           # AMax
    np.testing.assert_array_equal(sc(25, 1.0), np.where(np.abs(x) < 1, x, 1.0))                           # AMin
    np.testing.assert_allclose(sc(26, 2.0), np.arctan2(x, 2.0), rtol=1e-15)
    np.testing.assert_allclose(sc(31, 3.0), x ** 3, rtol=1e-14)                                           # Pow
    np.testing.assert_allclose(sc(45, 2.0), 2.0 ** x, rtol=1e-14)                                         # ReversePow
    np.testing.assert_array_equal(sc(34, 0.1), x * (1 - 0.1) + np.float64(np.float32(0.5)) * 0.1)         # SXELogitsSmoother
    np.testing.assert_array_equal(sc(35, 0.1), np.where(x < 0, 0.1 * x, x))                               # LeakyRELU
    np.testing.assert_array_equal(sc(36, 0.1), np.where(x >= 0, 1, 0.1))
    xp = np.abs(x) + 0.5
    np.testing.assert_allclose(sc(38, 2.0, xp), np.log2(xp), rtol=1e-14)                                  # LogX
    np.testing.assert_array_equal(sc(39, 0.0), np.maximum(x, 0))                                          # RELU
    np.testing.assert_array_equal(sc(40, 0.0), np.clip(x, 0, 6))                                          # RELU6
    np.testing.assert_array_equal(sc(41, 0.25), (x > 0.25).astype(np.float64))                            # Step
    np.testing.assert_array_equal(sc(49, 0.25), (x > 0.25).astype(np.float64))                            # RELUDerivative
    np.testing.assert_array_equal(sc(42, 2.0), np.clip(x, -2, 2))                                         # LstmClip
    np.testing.assert_array_equal(sc(43, 3.0), np.fmod(np.trunc(x), 3))                                   # TruncateMod
    np.testing.assert_array_equal(sc(46, 0.0), np.zeros_like(x))                                          # DivideNoNan
    np.testing.assert_array_equal(sc(13, 1.0), np.minimum(x, 1.0))
    np.testing.assert_array_equal(sc(6, 1.0), np.maximum(x, 1.0))


def test_scalar_takes_the_array_type_first():
    x = np.array([1.0, 2.0], np.float16)
    got = O.scalar(2, x, 0.1, np.zeros_like(x))                    # 0.1 becomes the nearest half first
    np.testing.assert_array_equal(got, (x.astype(np.float32) * np.float32(np.float16(0.1))).astype(np.float16))


@pytest.mark.parametrize("dims", [[0], [1], [2], [0, 2], [1, 2]])
def test_broadcast_runs_over_tads(dims):
    rng = np.random.default_rng(5)
    x = rng.uniform(-4, 4, (3, 4, 5))
    yshape = [x.shape[d] for d in dims]
    y = rng.uniform(0.5, 3, yshape)
    expand = [x.shape[d] if d in dims else 1 for d in range(3)]
    yb = y.reshape(expand)
    for op, fn in [(0, np.add), (1, np.subtract), (4, lambda a, b: b / a), (7, lambda a, b: np.power(np.abs(a), b)), (13, np.minimum),
                   (14, np.maximum), (17, lambda a, b: (a - b) ** 2), (18, np.mod), (19, lambda a, b: np.floor(a / b)), (22, np.mod),
                   (26, np.arctan2), (15, lambda a, b: np.where(np.abs(a) < np.abs(b), a, b)), (16, lambda a, b: np.where(np.abs(a) > np.abs(b), a, b))]:
        xx = np.abs(x) if op == 7 else x
        got = O.broadcast(op, xx, y, np.zeros_like(x), dims)
        np.testing.assert_allclose(got, fn(xx, yb) * np.ones_like(x), rtol=1e-14, atol=0, err_msg="op %d dims %s" % (op, dims))


def test_broadcast_on_views():
    rng = np.random.default_rng(6)
    base = rng.uniform(-1, 1, (5, 6, 4))
    x = base.transpose(2, 0, 1)                  # [4, 5, 6] view
    y = rng.uniform(1, 2, 5)
    got = O.broadcast(2, x, y, np.zeros((4, 5, 6)), [1])
    np.testing.assert_array_equal(got, x * y[None, :, None])


def test_entropy_reductions_match_scipy():
    import scipy.stats as stats
    rng = np.random.default_rng(3)
    p = rng.uniform(0.01, 1, (5, 64))
    p /= p.sum(1, keepdims=True)
    np.testing.assert_allclose(O.reduce_float(8, p, np.zeros(5), [1]), stats.entropy(p, axis=1), rtol=1e-13)
    np.testing.assert_allclose(O.reduce_float(9, p, np.zeros(5), [1]), np.log(stats.entropy(p, axis=1)), rtol=1e-13)
    np.testing.assert_allclose(O.reduce_float(10, p, np.zeros(5), [1]), stats.entropy(p, base=2, axis=1), rtol=1e-13)
    p32 = p.astype(np.float32)
    np.testing.assert_allclose(O.reduce_float(8, p32, np.zeros(5, np.float32), [1]), stats.entropy(p, axis=1), rtol=2e-6)
    np.testing.assert_allclose(O.reduce_float(10, p32.T.copy(), np.zeros(5, np.float32), [0]), stats.entropy(p, base=2, axis=1), rtol=2e-6)


def test_summary_stats_match_numpy_var_std():
    rng = np.random.default_rng(8)
    x = rng.normal(1000.0, 2.0, (6, 5, 40))          # large mean: a sum-of-squares formula would lose every digit
    for dims, axis in (([2], 2), ([0, 2], (0, 2)), (None, None)):
        shape = () if dims is None else tuple(s for i, s in enumerate(x.shape) if i not in dims)
        for bias in (False, True):
            v = O.summary_stats(0, x, np.zeros(shape), dims, bias)
            s = O.summary_stats(1, x, np.zeros(shape), dims, bias)
            np.testing.assert_allclose(v, np.var(x, axis=axis, ddof=int(bias)), rtol=1e-12)
            np.testing.assert_allclose(s, np.std(x, axis=axis, ddof=int(bias)), rtol=1e-12)
    one = np.array([[3.0], [4.0]])
    np.testing.assert_array_equal(O.summary_stats(0, one, np.zeros(2), [1], True), [0.0, 0.0])     # n <= 1 gives 0, not NaN
    x32 = x.astype(np.float32)
    np.testing.assert_allclose(O.summary_stats(0, x32, np.zeros((6, 5), np.float32), [2]), np.var(x32.astype(np.float64), axis=2), rtol=1e-6)


def test_counts_any_all_and_predicates():
    x = np.array([[0.0, 1.5, -2.0, 0.0], [0.0, 0.0, 0.0, 0.0], [1.0, 2.0, 3.0, -0.5], [-1.0, 1.0, 0.0, 0.0]])
    np.testing.assert_array_equal(O.reduce_long(0, x, np.zeros(4, np.int64), [1]), np.count_nonzero(x, axis=1))
    np.testing.assert_array_equal(O.reduce_long(1, x, np.zeros(4, np.int64), [1]), (x == 0).sum(1))
    np.testing.assert_array_equal(O.reduce_long(0, x, np.zeros((), np.int64)), np.count_nonzero(x))
    # Any is "the sum is positive" in the reference (ops.h:1200-1206): row 3 sums to 0 and row 0 to -0.5
    np.testing.assert_array_equal(O.reduce_bool(0, x, np.zeros(4, np.bool_), [1]), [False, False, True, False])
    np.testing.assert_array_equal(O.reduce_bool(1, x, np.zeros(4, np.bool_), [1]), [False, False, True, False])
    b = np.array([[True, False], [False, False], [True, True]])
    np.testing.assert_array_equal(O.reduce_bool(0, b, np.zeros(3, np.bool_), [1]), b.any(1))
    np.testing.assert_array_equal(O.reduce_bool(1, b, np.zeros(3, np.bool_), [1]), b.all(1))
    v = np.array([0.0, -0.0, 1.0, -3.0, np.inf, -np.inf, np.nan, 1e300])
    for op, fn in ((1, np.isinf), (2, np.isnan), (3, np.isfinite), (4, lambda a: ~np.isfinite(a)), (6, lambda a: a > 0), (7, lambda a: a == 0),
                   (8, lambda a: a < 0)):
        np.testing.assert_array_equal(O.transform_bool(op, v, np.zeros(v.shape, np.bool_)), fn(v), err_msg="op %d" % op)


def test_reduce3_reference_vectors_and_scipy():
    import scipy.spatial.distance as D
    # NDArrayTests.cpp:1473-1488 (applyReduce3EuclideanDistance is an all-pairs call; its diagonal is the pairwise result)
    x = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    y = np.full((2, 3), 2, np.float32)
    np.testing.assert_allclose(O.reduce3(1, x, y, np.zeros(2, np.float32), [1]), [1.414214, 5.385165], rtol=1e-6)
    # NDArrayTests2.cpp:1144-1152 reduce3_1
    np.testing.assert_array_equal(O.reduce3(1, np.array([[1, 2, 3, 4.0]]), np.array([[2, 3, 4, 5.0]]), np.zeros(4), [0]), [1, 1, 1, 1])
    rng = np.random.default_rng(9)
    a, b = rng.uniform(0.1, 2, (5, 40)), rng.uniform(0.1, 2, (5, 40))
    rows = lambda f: np.array([f(a[i], b[i]) for i in range(5)])
    z = lambda: np.zeros(5)
    np.testing.assert_allclose(O.reduce3(0, a, b, z(), [1]), rows(D.cityblock), rtol=1e-13)
    np.testing.assert_allclose(O.reduce3(1, a, b, z(), [1]), rows(D.euclidean), rtol=1e-13)
    np.testing.assert_allclose(O.reduce3(2, a, b, z(), [1]), 1 - rows(D.cosine), rtol=1e-12)
    np.testing.assert_allclose(O.reduce3(3, a, b, z(), [1]), (a * b).sum(1), rtol=1e-13)
    np.testing.assert_allclose(O.reduce3(5, a, b, z(), [1]), rows(D.cosine), rtol=1e-10, atol=1e-15)
    np.testing.assert_allclose(O.reduce3(6, a, b, z(), [1]), 1 - np.minimum(a, b).sum(1) / np.maximum(a, b).sum(1), rtol=1e-13)
    c = np.round(a)
    d = np.round(b)
    np.testing.assert_allclose(O.reduce3(7, c, d, z(), [1]), rows(lambda u, v: D.hamming(u, v)).astype(np.float64) * 0 + (c != d).mean(1), rtol=1e-15)
    np.testing.assert_allclose(O.reduce3(3, a, b, np.zeros(())), (a * b).sum(), rtol=1e-13)

"""Pins the numpy restatements of the remaining pairwise / scalar ops: the incomplete gamma functions against the values the
reference's own tests hold (libnd4j/tests_cpu/layers_tests/DeclarableOpsTests10.cpp:481-515) and scipy's library routine,
the others against closed forms a dropped term or a swapped operand would break."""
import numpy as np
import scipy.special

from oracle import oracle as O

A12 = np.array([1.1, 2.1, 3.1, 4.1, 5.1, 6.1, 7.1, 8.1, 9.1, 10.1, 11.1, 12.1]).reshape(1, 3, 4)
X4 = np.array([1.2, 2.2, 3.2, 4.2])
IGAMMA = np.array([0.659917, 0.61757898, 0.59726304, 0.58478117, 0.0066205109, 0.022211598, 0.040677428, 0.059117373,
                   0.0000039433403, 0.000086064574, 0.000436067, 0.0012273735]).reshape(1, 3, 4)
IGAMMAC = np.array([0.340083, 0.382421, 0.402737, 0.415221, 0.993379, 0.977788, 0.959323, 0.940883, 0.999996, 0.999914,
                    0.999564, 0.998773]).reshape(1, 3, 4)


def test_igamma_reference_vectors():
    np.testing.assert_allclose(O.igamma(A12, X4), IGAMMA, rtol=2e-5)                      # IGamma_Test1
    np.testing.assert_allclose(O.igamma(A12, X4, complement=True), IGAMMAC, rtol=2e-6)    # IGamma_Test2


def test_igamma_against_the_library_routine():
    rng = np.random.default_rng(5)
    a = rng.uniform(0.2, 8.0, 200)
    x = rng.uniform(0.05, 6.0, 200)
    # the reference stops the series when the running denominator passes 1e12, whatever x is: exact to rounding for small x,
    # short by up to a few 1e-4 relative once x reaches a few units
    small = x < 1.0
    np.testing.assert_allclose(O.igamma(a[small], x[small]), scipy.special.gammainc(a[small], x[small]), rtol=1e-9)
    np.testing.assert_allclose(O.igamma(a, x), scipy.special.gammainc(a, x), rtol=1e-3)
    assert (O.igamma(a, x) <= scipy.special.gammainc(a, x) * (1 + 1e-12)).all()            # a truncated series of positive terms
    np.testing.assert_allclose(O.igamma(a.astype(np.float32), x.astype(np.float32)), scipy.special.gammainc(a, x), rtol=1e-3)
    assert O.igamma(np.array([1e-7, 0.0, -1.0]), 2.0).tolist() == [0.0, 0.0, 0.0]           # the a <= 1e-6 guard
    np.testing.assert_allclose(O.igamma(np.array([1.0]), np.array([0.7])), 1 - np.exp(-0.7), rtol=1e-12)   # P(1, x) = 1 - e^-x


def test_relative_errors():
    x = np.array([0.0, 1.0, -1.0, 2.0, 1e-3, 5.0])
    y = np.array([0.0, 1.0, 1.0, 1.0, 2e-3, 5.000001])
    np.testing.assert_allclose(O.relative_error(x, y), [0.0, 0.0, 1.0, 1 / 3, 1 / 3, 1e-6 / 10.000001], rtol=1e-9)
    assert O.binary_relative_error(x, y, 0.1).tolist() == [0, 0, 1, 1, 1, 0]
    # the absolute threshold lets the tiny pair through: |1e-3 - 2e-3| < 0.01
    assert O.binary_min_abs_relative_error(x, y, 0.1, 0.01).tolist() == [0, 0, 1, 1, 0, 0]
    assert O.binary_min_abs_relative_error(x, y, 0.1, 1.5).tolist() == [0, 0, 1, 0, 0, 0]      # only |-1 - 1| = 2 stays above 1.5


def test_axpy_pow_derivative_log_poisson():
    x = np.array([1.0, 2.0, 3.0, 0.5])
    y = np.array([4.0, 3.0, 2.0, 1.0])
    assert O.axpy(x, y, 2.5).tolist() == [6.5, 8.0, 9.5, 2.25]
    np.testing.assert_allclose(O.pow_derivative(x, y), [4.0, 12.0, 6.0, 1.0])               # y x^(y-1)
    # d/dx x^y by central differences
    h = 1e-6
    np.testing.assert_allclose(O.pow_derivative(x, y), ((x + h) ** y - (x - h) ** y) / (2 * h), rtol=1e-6)
    np.testing.assert_allclose(O.log_poisson_loss(x, y), np.exp(y) - x * y)
    xs = np.array([1.0, 2.0, 3.0, 10.0])
    ys = np.array([0.3, -0.2, 1.0, 2.0])
    extra = O.log_poisson_loss(xs, ys, full=True) - O.log_poisson_loss(xs, ys)
    # Stirling: log x! = x log x - x + log(2 pi x) / 2 + 1 / (12 x) - ...
    gap = scipy.special.gammaln(xs + 1) - extra
    assert ((gap > 0) & (gap < 1 / (12 * xs))).all()
    np.testing.assert_allclose(extra[0], -1 + 0.5 * np.log(2 * np.pi), rtol=1e-12)

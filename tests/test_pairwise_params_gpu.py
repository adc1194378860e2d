"""The remaining pairwise / scalar opNums through the C ABI -- Axpy, RelativeError, the two thresholded relative errors,
PowDerivative, LogPoissonLoss(Full), IGamma / IGammac -- against the numpy restatements of oracle/oracle.py (pinned in
tests/test_oracle_pairwise_params.py) and the reference's own igamma vectors
(libnd4j/tests_cpu/layers_tests/DeclarableOpsTests10.cpp:481-515)."""
import numpy as np
import pytest

from deeplearning4j_amd.executioner import Pairwise, Scalar
from deeplearning4j_amd.nativeops import NativeOpsError
from deeplearning4j_amd.ndarray import DOUBLE, FLOAT32, HALF, NDArray
from oracle import oracle as O

pytestmark = pytest.mark.gpu

NP = {FLOAT32: np.float32, DOUBLE: np.float64, HALF: np.float16}
# tolerance of one library transcendental in the array's type
TOL = {DOUBLE: 1e-12, FLOAT32: 2e-6, HALF: 2e-3}


def _pair(rng, dt, shape=(53, 67)):
    return rng.uniform(0.25, 3.0, shape).astype(NP[dt]), rng.uniform(0.25, 3.0, shape).astype(NP[dt])


@pytest.mark.parametrize("dt", [DOUBLE, FLOAT32, HALF])
def test_relative_error_family(ex, dt):
    rng = np.random.default_rng(dt)
    x, y = _pair(rng, dt)
    y[::7] = x[::7]                     # equal pairs
    x[3, :5] = 0; y[3, :5] = 0          # two zeros: 0, not NaN
    y[5] = x[5] * NP[dt](1.0009765625)  # a relative error of about 5e-4
    X, Y = NDArray.from_numpy(x), NDArray.from_numpy(y)
    got = ex.exec_pairwise(Pairwise.RelativeError, X, Y).to_numpy()
    np.testing.assert_allclose(got.astype(np.float64), O.relative_error(x, y).astype(np.float64), rtol=TOL[dt] * 4, atol=0)
    assert not np.isnan(got).any()
    thr = 0.25
    got = ex.exec_pairwise(Pairwise.BinaryRelativeError, X, Y, extra_args=[thr]).to_numpy()
    want = O.binary_relative_error(x, y, thr)
    # a pair whose relative error sits within rounding of the threshold may fall on either side
    edge = np.abs(O.relative_error(x.astype(np.float64), y.astype(np.float64)) - thr) < 4 * TOL[dt]
    assert np.array_equal(got[~edge], want[~edge]) and set(np.unique(got)) <= {0.0, 1.0}
    got = ex.exec_pairwise(Pairwise.BinaryMinimumAbsoluteRelativeError, X, Y, extra_args=[thr, 1.0]).to_numpy()
    want = O.binary_min_abs_relative_error(x, y, thr, 1.0)
    edge |= np.abs(np.abs(x.astype(np.float64) - y.astype(np.float64)) - 1.0) < 4 * TOL[dt] * 3
    assert np.array_equal(got[~edge], want[~edge])
    assert want.sum() > 0 and want.sum() < O.binary_relative_error(x, y, thr).sum()      # the absolute threshold lets some through


@pytest.mark.parametrize("dt", [DOUBLE, FLOAT32, HALF])
def test_axpy(ex, dt):
    rng = np.random.default_rng(10 + dt)
    x, y = _pair(rng, dt, (41, 130))
    X, Y = NDArray.from_numpy(x), NDArray.from_numpy(y)
    got = ex.exec_pairwise(Pairwise.Axpy, X, Y, extra_args=[0.75]).to_numpy().astype(np.float64)
    # one fused multiply-add here, a multiply and an add in numpy: half a unit in the last place apart at most
    np.testing.assert_allclose(got, 0.75 * x.astype(np.float64) + y.astype(np.float64), rtol={DOUBLE: 3e-16, FLOAT32: 1.2e-7, HALF: 1e-3}[dt])
    # strided operands
    Xt = NDArray.from_numpy(np.ascontiguousarray(x.T)).permute(1, 0)
    got2 = ex.exec_pairwise(Pairwise.Axpy, Xt, Y, NDArray.empty(x.shape, dt), extra_args=[0.75]).to_numpy().astype(np.float64)
    assert np.array_equal(got2, got)
    with pytest.raises(NativeOpsError):
        ex.exec_pairwise(Pairwise.Axpy, X, Y)      # alpha is not optional


@pytest.mark.parametrize("dt", [DOUBLE, FLOAT32, HALF])
def test_pow_derivative_and_log_poisson(ex, dt):
    rng = np.random.default_rng(20 + dt)
    x, y = _pair(rng, dt)
    X, Y = NDArray.from_numpy(x), NDArray.from_numpy(y)
    f64 = lambda a: np.asarray(a).astype(np.float64)
    x64, y64 = f64(x), f64(y)
    tol = TOL[dt] * 8
    np.testing.assert_allclose(f64(ex.exec_pairwise(Pairwise.PowDerivative, X, Y).to_numpy()), y64 * x64 ** (y64 - 1), rtol=tol)
    np.testing.assert_allclose(f64(ex.exec_scalar(Scalar.PowDerivative, X, 2.5).to_numpy()), 2.5 * x64 ** 1.5, rtol=tol)
    np.testing.assert_allclose(f64(ex.exec_pairwise(Pairwise.LogPoissonLoss, X, Y).to_numpy()), f64(O.log_poisson_loss(x64, y64)), rtol=tol, atol=tol * 20)
    np.testing.assert_allclose(f64(ex.exec_pairwise(Pairwise.LogPoissonLossFull, X, Y).to_numpy()), f64(O.log_poisson_loss(x64, y64, full=True)), rtol=tol,
                               atol=tol * 20)


def test_igamma_reference_vectors(ex):
    a = np.array([1.1, 2.1, 3.1, 4.1, 5.1, 6.1, 7.1, 8.1, 9.1, 10.1, 11.1, 12.1]).reshape(3, 4)
    x = np.broadcast_to(np.array([1.2, 2.2, 3.2, 4.2]), (3, 4)).copy()
    want = np.array([0.659917, 0.61757898, 0.59726304, 0.58478117, 0.0066205109, 0.022211598, 0.040677428, 0.059117373,
                     0.0000039433403, 0.000086064574, 0.000436067, 0.0012273735]).reshape(3, 4)
    A, X = NDArray.from_numpy(a), NDArray.from_numpy(x)
    np.testing.assert_allclose(ex.exec_pairwise(Pairwise.IGamma, A, X).to_numpy(), want, rtol=2e-5)
    wantc = np.array([0.340083, 0.382421, 0.402737, 0.415221, 0.993379, 0.977788, 0.959323, 0.940883, 0.999996, 0.999914, 0.999564,
                      0.998773]).reshape(3, 4)
    np.testing.assert_allclose(ex.exec_pairwise(Pairwise.IGammac, A, X).to_numpy(), wantc, rtol=2e-6)


@pytest.mark.parametrize("dt,tol", [(DOUBLE, 1e-10), (FLOAT32, 2e-4)])
def test_igamma_against_the_restatement(ex, dt, tol):
    rng = np.random.default_rng(30 + dt)
    a = rng.uniform(0.2, 8.0, (17, 23)).astype(NP[dt])
    x = rng.uniform(0.05, 6.0, (17, 23)).astype(NP[dt])
    a[0, :3] = [1e-7, 0.0, -1.0]                                   # the a <= 1e-6 guard
    A, X = NDArray.from_numpy(a), NDArray.from_numpy(x)
    got = ex.exec_pairwise(Pairwise.IGamma, A, X).to_numpy()
    np.testing.assert_allclose(got.astype(np.float64), O.igamma(a, x).astype(np.float64), rtol=tol, atol=tol * 1e-3)
    assert got[0, :3].tolist() == [0.0, 0.0, 0.0]
    got = ex.exec_scalar(Scalar.IGamma, A, 1.5).to_numpy()
    np.testing.assert_allclose(got.astype(np.float64), O.igamma(a, 1.5).astype(np.float64), rtol=tol, atol=tol * 1e-3)
    got = ex.exec_scalar(Scalar.IGammac, A, 1.5).to_numpy()
    np.testing.assert_allclose(got.astype(np.float64), O.igamma(a, 1.5, complement=True).astype(np.float64), rtol=tol, atol=tol)


def test_broadcast_igamma_and_pow_derivative(ex):
    """Broadcast 32-34: the same functors with a row of second operands (the reference's IGamma_Test1 shape)."""
    from deeplearning4j_amd.executioner import Broadcast
    a = np.array([1.1, 2.1, 3.1, 4.1, 5.1, 6.1, 7.1, 8.1, 9.1, 10.1, 11.1, 12.1]).reshape(3, 4)
    x = np.array([1.2, 2.2, 3.2, 4.2])
    want = np.array([0.659917, 0.61757898, 0.59726304, 0.58478117, 0.0066205109, 0.022211598, 0.040677428, 0.059117373,
                     0.0000039433403, 0.000086064574, 0.000436067, 0.0012273735]).reshape(3, 4)
    A, X = NDArray.from_numpy(a), NDArray.from_numpy(x)
    np.testing.assert_allclose(ex.exec_broadcast(Broadcast.IGamma, A, X, [1]).to_numpy(), want, rtol=2e-5)
    np.testing.assert_allclose(ex.exec_broadcast(Broadcast.IGammac, A, X, [1]).to_numpy(), 1 - O.igamma(a, np.broadcast_to(x, a.shape)), rtol=1e-10)
    np.testing.assert_allclose(ex.exec_broadcast(Broadcast.PowDerivative, A, X, [1]).to_numpy(), x * a ** (x - 1), rtol=1e-12)


@pytest.mark.parametrize("dt", [DOUBLE, FLOAT32, HALF])
def test_reduce_bool_predicates(ex, dt):
    """ReduceBool 2-7 (ops/ops.h:1139-1163): true where any element of the sub-array is finite / inf or nan / nan / inf /
    positive / negative."""
    from deeplearning4j_amd.executioner import ReduceBool
    x = np.zeros((6, 40), NP[dt])
    x[1, 3] = np.nan
    x[2, 7] = -np.inf
    x[3, :] = np.nan            # nothing finite
    x[4, 11] = 2.0
    x[5, 39] = -0.5
    X = NDArray.from_numpy(x)
    fin = np.isfinite(x)
    want = {ReduceBool.IsFinite: fin.any(1), ReduceBool.IsInfOrNan: (~fin).any(1), ReduceBool.IsNan: np.isnan(x).any(1),
            ReduceBool.IsInf: np.isinf(x).any(1), ReduceBool.IsPositive: (x > 0).any(1), ReduceBool.IsNegative: (x < 0).any(1)}
    for op, w in want.items():
        assert np.array_equal(ex.exec_reduce_bool(op, X, [1]).to_numpy(), w), op
        assert bool(ex.exec_reduce_bool(op, X).to_numpy()) == bool(w.any()), op

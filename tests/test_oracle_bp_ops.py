"""Pins of the gradient-op restatements (softmax_bp, standardize, standardize_bp, layer_norm_bp, matmul_bp).

The reference's own tests for these ops hold shapes and all-zero cases only (DeclarableOpsTests15.cpp:72-90,397-408,
484-512); what fixes the values is the mathematics: each op must equal the central difference of the forward op's
restatement (itself pinned elsewhere), contracted with the incoming gradient."""
import numpy as np
import pytest

from oracle import oracle as o

H = 1e-6


def _numeric(f, x, g):
    num = np.zeros_like(x)
    for idx in np.ndindex(x.shape):
        xp, xm = x.copy(), x.copy()
        xp[idx] += H
        xm[idx] -= H
        num[idx] = np.sum((f(xp) - f(xm)) * g) / (2 * H)
    return num


def _softmax(x, dim):
    z = np.zeros_like(x)
    o.softmax(x, z, dim)
    return z


@pytest.mark.parametrize("shape,dim", [((4, 7), -1), ((3, 4, 5), 1), ((6,), 0), ((2, 3, 4), 0)])
def test_softmax_bp_is_the_derivative_of_softmax(shape, dim):
    rng = np.random.default_rng(7)
    x, g = rng.normal(0, 1, shape), rng.normal(0, 1, shape)
    got = o.softmax_bp(g, _softmax(x, dim), dim)
    assert np.abs(got - _numeric(lambda v: _softmax(v, dim), x, g)).max() < 1e-8
    # rows of a softmax sum to one, so the gradient rows sum to zero
    assert np.abs(got.sum(axis=dim)).max() < 1e-12


def test_standardize_reference_vector_and_closed_form():
    # DeclarableOpsTests15.cpp:72-81: a constant vector standardises to zeros
    assert np.array_equal(o.standardize(np.ones(5, np.float32), [0]), np.zeros(5, np.float32))
    rng = np.random.default_rng(8)
    x = rng.normal(2, 3, (3, 4, 5))
    z = o.standardize(x, [1, 2])
    assert np.abs(z.mean(axis=(1, 2))).max() < 1e-12
    assert np.abs(z.var(axis=(1, 2)) - x.var(axis=(1, 2)) / (x.var(axis=(1, 2)) + 1e-5)).max() < 1e-12


@pytest.mark.parametrize("shape,axes", [((3, 6), (1,)), ((2, 3, 4), (1, 2)), ((2, 3, 4), (0,)), ((5,), (0,))])
def test_standardize_bp_is_the_derivative_of_the_plain_z_score(shape, axes):
    rng = np.random.default_rng(9)
    x, g = rng.normal(0, 2, shape), rng.normal(0, 1, shape)
    f = lambda v: (v - v.mean(axis=axes, keepdims=True)) / v.std(axis=axes, keepdims=True)
    assert np.abs(o.standardize_bp(x, g, axes) - _numeric(f, x, g)).max() < 1e-7


def test_standardize_bp_constant_group_gives_zeros():
    # DeclarableOpsTests15.cpp:83-90 runs this case; 0/0 becomes NaN and NaN becomes 0 (standardize.cpp:148)
    assert np.array_equal(o.standardize_bp(np.ones(5, np.float32), np.zeros(5, np.float32), [0]), np.zeros(5, np.float32))
    assert np.array_equal(o.standardize_bp(np.ones(5, np.float32), np.arange(5, dtype=np.float32) - 2, [0]), np.zeros(5, np.float32))


def _layer_norm(x, gain, bias, axes, cf):
    z = np.zeros_like(x)
    o.layer_norm(x, gain, bias, z, list(axes), cf)
    return z


@pytest.mark.parametrize("shape,axes,cf", [((3, 4, 2, 2), (1, 2, 3), True), ((4, 6), (1,), False), ((2, 5, 3), (2,), False),
                                          ((2, 3, 4), (2,), True)])
def test_layer_norm_bp_matches_central_differences(shape, axes, cf):
    rng = np.random.default_rng(10)
    x, g = rng.normal(0, 2, shape), rng.normal(0, 1, shape)
    c = shape[1] if cf else shape[-1]
    gain, bias = rng.normal(1, 0.3, c), rng.normal(0, 0.3, c)
    dldx, dldg, dldb = o.layer_norm_bp(x, gain, g, axes, cf)
    # the forward op keeps 1e-5 inside the square root and the gradient op does not (standardize.cpp:62 against :103):
    # dLdx is the exact derivative of the epsilon-free z-score times gain
    bshape = [1] * x.ndim
    bshape[1 if cf else -1] = c
    plain = lambda v: (v - v.mean(axis=axes, keepdims=True)) / v.std(axis=axes, keepdims=True) * gain.reshape(bshape)
    num_x = _numeric(plain, x, g)
    assert np.abs(dldx - num_x).max() < 1e-7 * max(1.0, np.abs(num_x).max())
    num_g = _numeric(lambda v: _layer_norm(x, v, bias, axes, cf), gain, g)
    assert np.abs(dldg - num_g).max() < 1e-7 * max(1.0, np.abs(num_g).max())
    num_b = _numeric(lambda v: _layer_norm(x, gain, v, axes, cf), bias, g)
    assert np.abs(dldb - num_b).max() < 1e-7 * max(1.0, np.abs(num_b).max())


def test_layer_norm_bp_reference_cases():
    # DeclarableOpsTests15.cpp:484-494: zero eps gives zero gradients
    x = np.array([[1, 2, 3, 4, 5]], np.float32)
    g = np.array([1, 2, 3, 4, 5], np.float32)
    dldx, dldg, dldb = o.layer_norm_bp(x, g, np.zeros_like(x), [0], False)
    assert not dldx.any() and not dldg.any() and not dldb.any()
    # DeclarableOpsTests15.cpp:497-512 (shapes only there): axes {1,2,3}, channels first
    x = (-20 + 0.5 * np.arange(3 * 4 * 8 * 8)).reshape(3, 4, 8, 8).astype(np.float32)
    eps = (-4 + 0.05 * np.arange(3 * 4 * 8 * 8)).reshape(3, 4, 8, 8).astype(np.float32)
    dldx, dldg, dldb = o.layer_norm_bp(x, np.array([-0.1, 0.1, -0.2, 0.2], np.float32), eps, [1, 2, 3], True)
    assert dldx.shape == x.shape and dldg.shape == (4,) and dldb.shape == (4,)
    assert np.allclose(dldb, eps.sum(axis=(0, 2, 3)), rtol=1e-6)


@pytest.mark.parametrize("tx,ty,tz", [(0, 0, 0), (1, 0, 0), (0, 1, 0), (1, 1, 0), (0, 0, 1), (1, 1, 1)])
def test_matmul_bp_is_the_derivative_of_matmul(tx, ty, tz):
    rng = np.random.default_rng(11)
    a, b, c = 3, 4, 5
    x = rng.normal(0, 1, (b, a) if tx else (a, b))
    y = rng.normal(0, 1, (c, b) if ty else (b, c))
    zshape = (c, a) if tz else (a, c)
    g = rng.normal(0, 1, zshape)

    def fwd(xv, yv):
        z = np.zeros(zshape)
        o.matmul(xv, yv, z, bool(tx), bool(ty), bool(tz))
        return z
    dx, dy = o.matmul_bp(x, y, g, tx, ty, tz)
    assert np.abs(dx - _numeric(lambda v: fwd(v, y), x, g)).max() < 1e-8
    assert np.abs(dy - _numeric(lambda v: fwd(x, v), y, g)).max() < 1e-8


def test_matmul_bp_reference_shape_case():
    # DeclarableOpsTests15.cpp:397-408: a [1,3] (transposed), b [1,4], gradient [3,4]
    rng = np.random.default_rng(12)
    a, b, g = rng.normal(0, 1, (1, 3)), rng.normal(0, 1, (1, 4)), rng.normal(0, 1, (3, 4))
    dx, dy = o.matmul_bp(a, b, g, True, False, False)
    assert dx.shape == (1, 3) and dy.shape == (1, 4)
    assert np.allclose(dx, (g @ b.T).T) and np.allclose(dy, a @ g)

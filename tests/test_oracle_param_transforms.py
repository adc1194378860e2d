"""The two-parameter transforms of the oracle (clip_by_value, affine, scaled_tanh) against the reference's test vectors
and library routines."""
import numpy as np

from oracle import oracle as o


def _reference_clip_case():
    # DeclarableOpsTests1.cpp:801-848 (ClipByValue1 with T arguments, ClipByValue2 with scalar inputs): a 5x5 array of 4
    # with elements 0 and 1 set to -1 and 2, bounds [0, 3] -> 3 everywhere, 0 and 2 at the two elements
    x = np.full((5, 5), 4.0, np.float32)
    x.flat[0], x.flat[1] = -1.0, 2.0
    exp = np.full((5, 5), 3.0, np.float32)
    exp.flat[0], exp.flat[1] = 0.0, 2.0
    return x, exp


def test_clip_by_value_reference_vector():
    x, exp = _reference_clip_case()
    assert np.array_equal(o.clip_by_value(x, 0.0, 3.0), exp)


def test_clip_by_value_is_numpy_clip_and_keeps_nan():
    rng = np.random.default_rng(5)
    for dt in (np.float32, np.float64, np.float16):
        x = rng.normal(0, 2, (7, 33)).astype(dt)
        assert np.array_equal(o.clip_by_value(x, -1.25, 0.5), np.clip(x, dt(-1.25), dt(0.5)))
    x = np.array([np.nan, -np.inf, np.inf, 0.0], np.float32)
    got = o.clip_by_value(x, -1.0, 1.0)
    assert np.isnan(got[0]) and np.array_equal(got[1:], np.array([-1.0, 1.0, 0.0], np.float32))


def test_affine_and_scaled_tanh_closed_forms():
    rng = np.random.default_rng(6)
    x = rng.normal(0, 1, 1000)
    assert np.allclose(o.affine(x, 2.5, -0.75), 2.5 * x - 0.75, rtol=0, atol=1e-15)
    # a * tanh(b x) through exp: a * (e^{2bx} - 1) / (e^{2bx} + 1)
    e = np.exp(2 * 0.6666 * x)
    assert np.allclose(o.scaled_tanh(x, 1.7159, 0.6666), 1.7159 * (e - 1) / (e + 1), rtol=1e-12, atol=1e-14)
    # odd in x, bounded by |a|, slope a*b at the origin
    assert np.allclose(o.scaled_tanh(-x, 1.7159, 0.6666), -o.scaled_tanh(x, 1.7159, 0.6666))
    assert np.abs(o.scaled_tanh(50 * x, 1.7159, 0.6666)).max() <= 1.7159
    h = 1e-6
    assert abs(o.scaled_tanh(np.array([h]), 1.7159, 0.6666)[0] / h - 1.7159 * 0.6666) < 1e-6


def test_stabilize_and_set_range_hand_cases():
    cut = float(np.float32(3.79297773665))
    x = np.array([0.5, 2.0, -2.0, 1.8, -1.9], np.float64)
    # k = 2: x*k = 1, 4, -4, 3.6, -3.8 -> inside, above, below, inside, below
    got = o.stabilize(x, 2.0)
    assert np.allclose(got, [0.5, cut / 2, -cut / 2, 1.8, -cut / 2], rtol=0, atol=1e-15)
    # the result times k never leaves the cutoff, and values inside are untouched
    rng = np.random.default_rng(8)
    y = rng.normal(0, 5, 1000)
    assert (np.abs(o.stabilize(y, 0.7) * 0.7) <= cut * (1 + 1e-12)).all()
    inside = np.abs(y * 0.7) <= cut
    assert np.array_equal(o.stabilize(y, 0.7)[inside], y[inside])
    # SetRange: inside stays; outside the unit range goes through a sigmoid and floors to 0; another range floors x * width + lo
    z = np.array([0.25, 1.0, 3.0, -3.0], np.float64)
    assert np.array_equal(o.set_range(z, 0.0, 1.0), [0.25, 1.0, 0.0, 0.0])
    assert np.array_equal(o.set_range(np.array([2.5, 7.25, -1.5]), 2.0, 4.0), [2.5, np.floor(7.25 * 2) + 2, np.floor(-1.5 * 2) + 2])

"""The oracle's strided_slice against the reference's own test vectors (tests/golden/strided_slice_vectors.json) and
against element-by-element brute force; the other shape ops against hand-checkable cases (CPU only)."""
import itertools
import json
import os

import numpy as np
import pytest

from oracle import oracle as O

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "strided_slice_vectors.json")))["cases"]


def _specs(case):
    if "iargs" in case:
        v = case["iargs"]
        n = len(v) // 3
        return v[:n], v[n:2 * n], v[2 * n:]
    i = case["inputs"]
    return i["begin"], i["end"], i["strides"]


@pytest.mark.parametrize("case", GOLD, ids=[c["name"].split()[-1] for c in GOLD])
def test_strided_slice_reference_vectors(case):
    x = np.array(case["x"], dtype=np.float64)
    b, e, s = _specs(case)
    got = O.strided_slice(x, b, e, s, *case["masks"])
    assert list(got.shape) == case["shape"]
    np.testing.assert_array_equal(got.reshape(-1), np.array(case["exp"], dtype=np.float64))


def test_strided_slice_brute_force_including_negative_steps():
    x = np.arange(4 * 5 * 6).reshape(4, 5, 6)
    rng = np.random.default_rng(0)
    for _ in range(200):
        b = [int(rng.integers(-7, 8)) for _ in range(3)]
        e = [int(rng.integers(-7, 8)) for _ in range(3)]
        s = [int(rng.choice([-3, -2, -1, 1, 2, 3])) for _ in range(3)]
        got = O.strided_slice(x, b, e, s)
        # element-by-element: python's range() is the definition of a clamped strided walk
        axes = [range(*slice(b[d], e[d], s[d]).indices(x.shape[d])) for d in range(3)]
        want = np.array([x[i, j, k] for i, j, k in itertools.product(*axes)]).reshape([len(a) for a in axes])
        np.testing.assert_array_equal(got, want)


def test_other_shape_ops():
    x = np.arange(24.0).reshape(2, 3, 4)
    p = O.permute(x, [2, 0, 1])
    assert p.shape == (4, 2, 3) and p[3, 1, 2] == x[1, 2, 3] and p.flags.c_contiguous
    assert O.permute(x).shape == (4, 3, 2) and O.permute(x)[3, 2, 1] == x[1, 2, 3]
    r = O.reshape(x, [4, -1])
    assert r.shape == (4, 6) and r[1, 0] == 6.0
    rf = O.reshape(x, [4, 6], "f")
    # column-major sequence of x: x[0,0,0], x[1,0,0], x[0,1,0], ... lands column-major in the result
    assert rf[0, 0] == x[0, 0, 0] and rf[1, 0] == x[1, 0, 0] and rf[2, 0] == x[0, 1, 0] and rf[0, 1] == x[0, 2, 0]
    y = x.reshape(2, 1, 3, 1, 4)
    assert O.squeeze(y).shape == (2, 3, 4) and O.squeeze(y, [1]).shape == (2, 3, 1, 4) and O.squeeze(y, [0, 3]).shape == (2, 1, 3, 4)
    assert O.expand_dims(x, 1).shape == (2, 1, 3, 4) and O.expand_dims(x, -1).shape == (2, 3, 4, 1)
    parts = O.split(x, 2, axis=2)
    assert len(parts) == 2 and parts[1].shape == (2, 3, 2) and parts[1][1, 2, 0] == x[1, 2, 2]

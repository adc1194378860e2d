"""The log_softmax restatement against the reference's own test vectors (tests/golden/log_softmax_vectors.json)."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as o

CASES = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "log_softmax_vectors.json")))["cases"]


@pytest.mark.parametrize("case", CASES, ids=[c["name"].split()[-1] for c in CASES])
def test_log_softmax_reference_vectors(case):
    x = np.array(case["x"], np.float64).reshape(case["shape"])
    dim = case["iargs"][0] if case["iargs"] else x.ndim - 1
    got = o.log_softmax(x, dim)
    want = np.array(case["exp"], np.float64).reshape(case["shape"])
    # the expected arrays carry six significant digits
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=2e-5, atol=case.get("tol", 1e-5))


def test_log_softmax_underflow_is_minus_infinity_as_in_the_reference():
    x = np.array([[0.0, -200.0, 1.0]], np.float32)
    got = o.log_softmax(x, 1)
    assert np.isneginf(got[0, 1]) and np.isfinite(got[0, [0, 2]]).all()

import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.build()
    return O


@pytest.fixture(scope="session")
def ex():
    """The executioner over libnd4jhip.so; fails loudly when the library or the GPU is missing."""
    from deeplearning4j_amd.executioner import Executioner
    return Executioner()


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)["cases"]


def materialize(spec):
    """Fixture array -> numpy array with the logical values, laid out in the order the fixture names."""
    dt = np.dtype(spec["dtype"] or "float64")
    shape = spec["shape"]
    if "buffer" in spec:
        a = np.array(spec["buffer"], dtype=np.float64).reshape(shape, order="F" if spec["order"] == "f" else "C")
    else:
        a = np.array(spec["logical"], dtype=np.float64).reshape(shape)
    a = a.astype(dt)
    if a.ndim == 0:
        return a
    return np.asfortranarray(a) if spec["order"] == "f" and a.ndim > 1 else np.ascontiguousarray(a)


def assert_close(actual, expected, rtol, atol, what=""):
    """|a - b| <= atol + rtol * |b| elementwise, with a readable report."""
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    assert actual.shape == expected.shape, "%s: shape %s vs %s" % (what, actual.shape, expected.shape)
    err = np.abs(actual - expected)
    bound = atol + rtol * np.abs(expected)
    bad = ~(err <= bound)
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err - bound, -np.inf)), err.shape) if err.ndim else ()
        raise AssertionError("%s: %d of %d elements out of tolerance (rtol %g, atol %g); worst at %s: got %r, want %r"
                             % (what, int(bad.sum()), err.size, rtol, atol, i, actual[i], expected[i]))

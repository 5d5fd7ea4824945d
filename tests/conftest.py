import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
PY_HOST = os.path.join(ROOT, "tfjs-core_amd", "python")
if PY_HOST not in sys.path:
    sys.path.insert(0, PY_HOST)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


_cache = {}


def golden_case(fixture, title, describe=None):
    """One case of a fixture written by tests/golden/extract_golden.py."""
    if fixture not in _cache:
        with open(os.path.join(GOLDEN, fixture + ".json")) as f:
            _cache[fixture] = json.load(f)
    for c in _cache[fixture]["cases"]:
        if c["title"] == title and (describe is None or c["describe"] == describe):
            return c
    raise KeyError((fixture, describe, title))


def golden_cases(fixture):
    """All cases of a fixture, in the order of the reference's test file."""
    if fixture not in _cache:
        with open(os.path.join(GOLDEN, fixture + ".json")) as f:
            _cache[fixture] = json.load(f)
    return _cache[fixture]["cases"]


def f32(a, shape=None):
    x = np.array(a, dtype=np.float32)
    return x.reshape(shape) if shape is not None else x


def expect_close(actual, expected, eps=1e-3):
    """expectArraysClose of the reference (test_util.ts:22-39,121-138): absolute epsilon
    1e-3 on a 32-bit backend; NaN matches NaN."""
    a = np.asarray(actual, dtype=np.float64).ravel()
    e = np.asarray(expected, dtype=np.float64).ravel()
    assert a.shape == e.shape, (a.shape, e.shape)
    both_nan = np.isnan(a) & np.isnan(e)
    same_inf = np.isinf(a) & np.isinf(e) & (np.sign(a) == np.sign(e))
    ok = both_nan | same_inf | (np.abs(a - e) <= eps)
    assert ok.all(), "mismatch at %s: actual %s expected %s" % (
        np.nonzero(~ok)[0][:8], a[~ok][:8], e[~ok][:8])


@pytest.fixture(scope="session")
def oracle():
    from oracle import cpu_ref
    cpu_ref.build()
    return cpu_ref

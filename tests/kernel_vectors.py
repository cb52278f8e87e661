"""The known-answer vectors of the reference's kernel crate (cuda/src/kernels/*.rs #[test]s), as
tests/golden/extract_reference_cases.py wrote them to tests/golden/reference_cases.json, and the
comparison rules of the assertion macros those tests use."""
import json
import os

import numpy as np

from optest import decode

HERE = os.path.dirname(os.path.abspath(__file__))
KERNEL_CASES = json.load(open(os.path.join(HERE, "golden", "reference_cases.json")))["kernel_cases"]


def ids(cases):
    return [c["test"] for c in cases]


def arr(case, key, dtype_key="dtype", shape=None):
    a = decode(case[key], case[dtype_key])
    return a.reshape(shape) if shape is not None else a


def check(actual, expected, compare="exact", epsilon=0.0):
    """assert_eq! ("exact"), approx::assert_relative_eq! ("relative": |a-e| <= epsilon, or
    <= max(|a|,|e|) * the type's machine epsilon) and approx::assert_abs_diff_eq! ("abs_diff")."""
    actual = np.asarray(actual).reshape(-1)
    expected = np.asarray(expected).reshape(-1)
    assert actual.shape == expected.shape, (actual.shape, expected.shape)
    assert actual.dtype == expected.dtype, (actual.dtype, expected.dtype)
    if compare == "exact" or actual.dtype.kind != "f":
        nan = (actual != actual) & (expected != expected) if actual.dtype.kind == "f" else np.zeros(actual.shape, bool)
        assert np.array_equal(actual[~nan], expected[~nan]), (actual, expected)
        return
    a, e = actual.astype(np.float64), expected.astype(np.float64)
    diff = np.abs(a - e)
    ok = diff <= epsilon
    if compare == "relative":
        ok |= diff <= np.maximum(np.abs(a), np.abs(e)) * float(np.finfo(actual.dtype).eps)
    assert ok.all(), (actual, expected, epsilon)

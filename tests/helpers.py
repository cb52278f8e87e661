"""Shared helpers for the parity tests."""
import numpy as np


def bcast_strides(shape, out_shape):
    """Element stride of `shape` per output dim, 0 on broadcast dims (the meaning of the
    reference's info buffers, runtime/src/utils/mod.rs:56-112)."""
    shape = list(shape)
    dense = [0] * len(shape)
    acc = 1
    for i in range(len(shape) - 1, -1, -1):
        dense[i] = acc
        acc *= shape[i]
    n = len(out_shape)
    out = [0] * n
    for i in range(n):
        j = i - (n - len(shape))
        if j >= 0 and shape[j] == out_shape[i] and shape[j] != 1:
            out[i] = dense[j]
    return out


def to_dev(arr, device):
    import torch
    arr = np.ascontiguousarray(arr)
    if arr.dtype == np.bool_:
        return torch.from_numpy(arr.astype(np.uint8)).to(device).view(torch.bool)
    return torch.from_numpy(arr).to(device)


def to_np(t):
    import torch
    if t.dtype == torch.bool:
        return t.view(torch.uint8).cpu().numpy().astype(np.bool_)
    return t.cpu().numpy()


def assert_close(actual, expected, rtol=1e-4, atol=1e-5):
    """The reference's per-op acceptance: abs(a - e) <= atol + rtol * abs(e), NaN == NaN,
    equal infinities (runtime/tests/onnx_node/main.rs:26-27,304-311)."""
    actual = np.asarray(actual)
    expected = np.asarray(expected)
    assert actual.shape == expected.shape, (actual.shape, expected.shape)
    assert actual.dtype == expected.dtype, (actual.dtype, expected.dtype)
    np.testing.assert_allclose(actual, expected, rtol=rtol, atol=atol, equal_nan=True)


def assert_exact(actual, expected):
    actual = np.asarray(actual)
    expected = np.asarray(expected)
    assert actual.shape == expected.shape, (actual.shape, expected.shape)
    assert actual.dtype == expected.dtype, (actual.dtype, expected.dtype)
    if actual.dtype.kind == "f":
        # bit-exact, NaN payloads included
        bits = {2: np.uint16, 4: np.uint32, 8: np.uint64}[actual.dtype.itemsize]
        a = np.ascontiguousarray(actual).view(bits)
        e = np.ascontiguousarray(expected).view(bits)
        both_nan = np.isnan(actual) & np.isnan(expected)
        assert np.array_equal(a[~both_nan], e[~both_nan])
    else:
        assert np.array_equal(actual, expected)

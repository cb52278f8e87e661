"""Error behaviour of the C-ABI entry points of the kernel rows: a call with arguments the header
rules out answers with the documented status and launches nothing (the output keeps its canary
bytes), like the reference's kernel wrappers, which return Err before they launch
(cuda/src/kernels/binary.rs:93-102 "unsupported data type", gemm.rs:191-232, slice.rs:61-122)."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

OK, BAD_RANK, UNSUPPORTED, NULL_POINTER, SIZE_MISMATCH, INVALID_ARGUMENT = 0, -1, -2, -3, -4, -5
TOO_LARGE = -7


@pytest.fixture(scope="module")
def env():
    import torch
    from rmlk_amd import kernels as k
    from rmlk_amd._lib import Dims, lib
    dev = torch.device("cuda:0")
    a = torch.arange(64, dtype=torch.float32, device=dev)
    b = torch.arange(64, dtype=torch.float32, device=dev) + 100
    out = torch.full((64,), -7.0, dtype=torch.float32, device=dev)
    idx = torch.zeros(8, dtype=torch.int64, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    return dict(torch=torch, k=k, L=lib(), D=Dims.of, a=a, b=b, out=out, idx=idx, flag=flag,
                stream=torch.cuda.current_stream().cuda_stream)


def _untouched(env):
    env["torch"].cuda.synchronize()
    assert bool((env["out"] == -7.0).all()), "a rejected call wrote to its output"
    assert int(env["flag"].item()) == 0


def p(t):
    return ctypes.c_void_p(t.data_ptr())


NULL = ctypes.c_void_p(0)


def test_binary_where(env):
    L, D, k, s = env["L"], env["D"], env["k"], env["stream"]
    a, b, out = p(env["a"]), p(env["b"]), p(env["out"])
    shape, dense = D([4, 16]), D([16, 1])
    nine = D([1] * 8)
    nine.rank = 9
    zero = D([1])
    zero.rank = 0
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.FLOAT, nine, dense, dense, a, b, out) == BAD_RANK
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.FLOAT, zero, dense, dense, a, b, out) == BAD_RANK
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.FLOAT, None, dense, dense, a, b, out) == BAD_RANK
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.FLOAT, shape, D([1]), dense, a, b, out) == SIZE_MISMATCH
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.FLOAT, D([4, -1]), dense, dense, a, b, out) == INVALID_ARGUMENT
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.FLOAT, shape, D([-16, 1]), dense, a, b, out) == INVALID_ARGUMENT
    for args in ((NULL, b, out), (a, NULL, out), (a, b, NULL)):
        assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.FLOAT, shape, dense, dense, *args) == NULL_POINTER
    # an empty output asks for nothing, also of null pointers
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.FLOAT, D([0, 16]), dense, dense, NULL, NULL, NULL) == OK
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.INT32, shape, dense, dense, a, b, out) == UNSUPPORTED
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT16, k.FLOAT16, shape, dense, dense, a, b, out) == UNSUPPORTED
    assert L.rmlk_hip_binary(s, 99, k.FLOAT, k.FLOAT, shape, dense, dense, a, b, out) != OK
    cond_t = env["torch"].ones(64, dtype=env["torch"].bool, device=env["a"].device)
    cond = p(cond_t)
    assert L.rmlk_hip_where(s, k.FLOAT, nine, dense, dense, dense, a, b, cond, out) == BAD_RANK
    assert L.rmlk_hip_where(s, k.FLOAT, shape, dense, D([1]), dense, a, b, cond, out) == SIZE_MISMATCH
    assert L.rmlk_hip_where(s, k.FLOAT, shape, dense, dense, dense, a, b, NULL, out) == NULL_POINTER
    assert L.rmlk_hip_where(s, k.FLOAT, shape, dense, dense, D([16, -1]), a, b, cond, out) == INVALID_ARGUMENT
    _untouched(env)


def test_maps_and_reductions(env):
    L, D, k, s = env["L"], env["D"], env["k"], env["stream"]
    a, out = p(env["a"]), p(env["out"])
    assert L.rmlk_hip_unary(s, k.SQRT, k.FLOAT, -1, a, out) == INVALID_ARGUMENT
    assert L.rmlk_hip_unary(s, 17, k.FLOAT, 64, a, out) == INVALID_ARGUMENT
    assert L.rmlk_hip_unary(s, k.SQRT, k.INT32, 64, a, out) == UNSUPPORTED     # "unsupported data type"
    assert L.rmlk_hip_unary(s, k.SQRT, k.FLOAT, 64, NULL, out) == NULL_POINTER
    assert L.rmlk_hip_unary(s, k.SQRT, k.FLOAT, 1 << 62, a, out) == TOO_LARGE
    assert L.rmlk_hip_unary(s, k.SQRT, k.FLOAT, 0, NULL, NULL) == OK
    assert L.rmlk_hip_cast(s, k.FLOAT, 99, 64, a, out) == UNSUPPORTED
    assert L.rmlk_hip_cast(s, k.FLOAT, k.INT32, -3, a, out) == INVALID_ARGUMENT
    assert L.rmlk_hip_cast(s, k.FLOAT, k.INT32, 64, a, NULL) == NULL_POINTER
    axes = (ctypes.c_int64 * 2)(1, 1)
    one = (ctypes.c_int64 * 1)(2)
    assert L.rmlk_hip_reduce_mean(s, k.FLOAT, D([4, 16]), axes, 2, a, out) == INVALID_ARGUMENT   # an axis twice
    assert L.rmlk_hip_reduce_mean(s, k.FLOAT, D([4, 16]), one, 1, a, out) == INVALID_ARGUMENT    # axis == rank
    assert L.rmlk_hip_reduce_mean(s, k.FLOAT, D([4, 16]), None, 1, a, out) == NULL_POINTER
    assert L.rmlk_hip_reduce_mean(s, k.INT32, D([4, 16]), axes, 1, a, out) == UNSUPPORTED
    assert L.rmlk_hip_reduce_mean(s, k.FLOAT, D([4, 16]), axes, 0, a, out) == INVALID_ARGUMENT
    assert L.rmlk_hip_reduce_mean(s, k.FLOAT, D([4, 16]), axes, 1, NULL, out) == NULL_POINTER
    assert L.rmlk_hip_softmax(s, k.INT64, 4, 16, 1, a, out) == UNSUPPORTED
    assert L.rmlk_hip_softmax(s, k.FLOAT, 4, -16, 1, a, out) == INVALID_ARGUMENT
    assert L.rmlk_hip_softmax(s, k.FLOAT, 4, 16, 1, a, NULL) == NULL_POINTER
    assert L.rmlk_hip_softmax(s, k.FLOAT, 1 << 40, 1 << 30, 1, a, out) == TOO_LARGE
    assert L.rmlk_hip_softmax(s, k.FLOAT, 0, 16, 1, NULL, NULL) == OK
    _untouched(env)


def test_matmul(env):
    L, k, s = env["L"], env["k"], env["stream"]
    a, b, out = p(env["a"]), p(env["b"]), p(env["out"])

    def mm(dtype=k.FLOAT, batch=1, m=4, n=4, kk=4, pa=a, lda=4, sa=0, pb=b, ldb=4, sb=0, pc=out, ldc=4, sc=0):
        return L.rmlk_hip_matmul(s, dtype, batch, m, n, kk, pa, lda, sa, 0, pb, ldb, sb, 0, pc, ldc, sc, NULL, 0)

    assert mm(dtype=k.DOUBLE) == UNSUPPORTED
    assert mm(m=-1) == INVALID_ARGUMENT
    assert mm(sa=-16) == INVALID_ARGUMENT
    assert mm(pa=NULL) == NULL_POINTER
    assert mm(pc=NULL) == NULL_POINTER
    assert mm(lda=3) == SIZE_MISMATCH          # leading dimension shorter than a row
    assert mm(ldc=2) == SIZE_MISMATCH
    assert mm(batch=70000) == TOO_LARGE
    assert mm(m=0, pa=NULL, pb=NULL, pc=NULL) == OK
    _untouched(env)


def test_movement(env):
    L, D, k, s = env["L"], env["D"], env["k"], env["stream"]
    a, out, idx, flag = p(env["a"]), p(env["out"]), p(env["idx"]), p(env["flag"])
    perm_twice = (ctypes.c_int64 * 2)(0, 0)
    perm_far = (ctypes.c_int64 * 2)(0, 2)
    perm = (ctypes.c_int64 * 2)(1, 0)
    assert L.rmlk_hip_transpose(s, k.FLOAT, D([4, 16]), perm_twice, a, out) == INVALID_ARGUMENT
    assert L.rmlk_hip_transpose(s, k.FLOAT, D([4, 16]), perm_far, a, out) == INVALID_ARGUMENT
    assert L.rmlk_hip_transpose(s, k.FLOAT, D([4, 16]), None, a, out) == NULL_POINTER
    assert L.rmlk_hip_transpose(s, 99, D([4, 16]), perm, a, out) == UNSUPPORTED
    assert L.rmlk_hip_transpose(s, k.FLOAT, D([4, 16]), perm, a, NULL) == NULL_POINTER
    assert L.rmlk_hip_expand(s, k.FLOAT, D([3, 16]), D([4, 16]), a, out) == SIZE_MISMATCH     # 3 does not repeat to 4
    assert L.rmlk_hip_expand(s, k.FLOAT, D([1, 4, 16]), D([4, 16]), a, out) == SIZE_MISMATCH  # input of higher rank
    assert L.rmlk_hip_expand(s, k.FLOAT, D([1, 16]), D([4, 16]), NULL, out) == NULL_POINTER
    sl = lambda starts, steps, shape: L.rmlk_hip_slice(s, k.FLOAT, D([4, 16]), D(starts), D(steps), D(shape), a, out)
    assert sl([0, 0], [1, 0], [4, 4]) == INVALID_ARGUMENT      # step 0 (ref: ZeroStep)
    assert sl([0, 16], [1, 1], [4, 1]) == INVALID_ARGUMENT     # start past the end
    assert sl([0, 8], [1, 1], [4, 9]) == INVALID_ARGUMENT      # runs past the end
    assert sl([0, 3], [1, -1], [4, 5]) == INVALID_ARGUMENT     # runs below 0
    assert sl([0], [1], [4]) == SIZE_MISMATCH
    cc = lambda in_shape, out_shape, axis, off: L.rmlk_hip_concat(s, k.FLOAT, D(in_shape), D(out_shape), axis, off, a, out)
    assert cc([2, 16], [4, 16], 2, 0) == INVALID_ARGUMENT
    assert cc([2, 8], [4, 16], 0, 0) == SIZE_MISMATCH           # other dims differ
    assert cc([2, 16], [3, 16], 0, 2) == SIZE_MISMATCH          # past the end of the axis
    assert cc([2, 16], [4, 16], 0, -1) == SIZE_MISMATCH
    ga = lambda dtype, idt, axis, n, data, ix, o: L.rmlk_hip_gather(s, dtype, idt, D([4, 16]), axis, n, data, ix, o, flag)
    assert ga(k.FLOAT, k.INT64, 2, 2, a, idx, out) == INVALID_ARGUMENT
    assert ga(k.FLOAT, k.FLOAT, 0, 2, a, idx, out) == UNSUPPORTED     # index type
    assert ga(k.FLOAT, k.INT64, 0, -2, a, idx, out) == INVALID_ARGUMENT
    assert ga(k.FLOAT, k.INT64, 0, 2, a, NULL, out) == NULL_POINTER
    assert ga(k.FLOAT, k.INT64, 0, 2, NULL, idx, out) == NULL_POINTER
    sc = lambda red, dtype, n, tuple_size, ix, upd, o: L.rmlk_hip_scatter_nd(s, red, dtype, D([4, 16]), n, tuple_size, ix, upd, o, flag)
    assert sc(0, k.FLOAT, 2, 3, idx, a, out) == INVALID_ARGUMENT       # tuple longer than the rank
    assert sc(0, k.FLOAT, 2, 0, idx, a, out) == INVALID_ARGUMENT
    assert sc(9, k.FLOAT, 2, 1, idx, a, out) == INVALID_ARGUMENT       # no such reduction
    assert sc(1, k.BOOL, 2, 1, idx, a, out) == UNSUPPORTED             # add over booleans
    assert sc(0, k.FLOAT, -1, 1, idx, a, out) == INVALID_ARGUMENT
    assert sc(0, k.FLOAT, 2, 1, NULL, a, out) == NULL_POINTER
    assert sc(0, k.FLOAT, 0, 1, NULL, NULL, NULL) == OK
    tr = lambda dtype, batch, rows, cols, i, o: L.rmlk_hip_trilu(s, dtype, batch, rows, cols, 1, 0, i, o)
    assert tr(99, 1, 4, 16, a, out) == UNSUPPORTED
    assert tr(k.FLOAT, 1, -4, 16, a, out) == INVALID_ARGUMENT
    assert tr(k.FLOAT, 1, 4, 16, a, NULL) == NULL_POINTER
    assert tr(k.FLOAT, 1 << 40, 1 << 30, 16, a, out) == TOO_LARGE
    many = L.rmlk_hip_memcpy_dtod_many
    assert many(s, -1, None, None, None) == INVALID_ARGUMENT
    assert many(s, 2, None, None, None) == NULL_POINTER
    assert many(s, 0, None, None, None) == OK
    _untouched(env)


def test_a_good_call_after_the_rejected_ones(env):
    """The library keeps no error state: the call after a rejected one runs."""
    L, D, k, s = env["L"], env["D"], env["k"], env["stream"]
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.FLOAT, D([4, 16]), D([16, 1]), D([16, 1]), NULL, NULL, NULL) == NULL_POINTER
    assert L.rmlk_hip_binary(s, k.ADD, k.FLOAT, k.FLOAT, D([4, 16]), D([16, 1]), D([0, 1]), p(env["a"]), p(env["b"]),
                             p(env["out"])) == OK
    env["torch"].cuda.synchronize()
    got = env["out"].cpu().numpy().reshape(4, 16)
    exp = np.arange(64, dtype=np.float32).reshape(4, 16) + (np.arange(16, dtype=np.float32) + 100)
    assert np.array_equal(got, exp)
    env["out"].fill_(-7.0)

"""rmlk_hip_matmul_noalloc (split-K partials in the library's fixed device array) against
rmlk_hip_matmul (partials in a workspace the caller allocates): the same kernels write the same
partials in the same order, so the results are held to bit equality, and to the float64 oracle
within the fp32 MatMul bar (rtol 1e-4 / atol 1e-5 scaled by the K-long sum).

The array keeps the last call's contents, so every case makes two calls in a row through the C ABI,
the second with a smaller problem that reuses the front of the array.
"""
import numpy as np
import pytest

from helpers import assert_exact

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

SCRATCH_BYTES = 32 << 20   # RMLK_HIP_MATMUL_NOALLOC_SCRATCH_BYTES in include/rmlk_hip.h


def _both(device, rng, batch, m, n, k, trans_b=False, b_broadcast=False):
    from rmlk_amd import kernels as kk
    from oracle import ops
    a = rng.standard_normal((batch, m, k), dtype=np.float32)
    nb = 1 if b_broadcast else batch
    b = (rng.standard_normal((nb, n, k) if trans_b else (nb, k, n), dtype=np.float32) * 0.05).astype(np.float32)
    da, db = torch.from_numpy(a).to(device), torch.from_numpy(b).to(device)
    ldb = k if trans_b else n
    stride_b = 0 if b_broadcast else n * k
    # the first call of the entry point on a device looks its array up (and, in a fresh process, has
    # the code object loaded): done here, outside the measurement of free memory
    w = torch.zeros(8, 8, device=device)
    kk.matmul_noalloc(w, w, torch.empty(8, 8, device=device), 1, 8, 8, 8, 8, 8, 8, 64, 64, 64)
    torch.cuda.synchronize()
    outs = []
    for fn in (kk.matmul, kk.matmul_noalloc):
        c = torch.full((batch, m, n), float("nan"), device=device)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        fn(da, db, c, batch, m, n, k, k, ldb, n, m * k, stride_b, m * n, False, trans_b)
        torch.cuda.synchronize()
        if fn is kk.matmul_noalloc:
            # device memory in use did not change across the call
            assert torch.cuda.mem_get_info()[0] == free_before
        outs.append(c.cpu().numpy())
    assert_exact(outs[1], outs[0])
    bb = np.swapaxes(b, -1, -2) if trans_b else b
    ref = ops.matmul(a, bb)
    np.testing.assert_allclose(outs[1], ref, rtol=1e-4, atol=1e-5 * np.sqrt(k) * 4)
    return kk.matmul_workspace_size(batch, m, n, k)


# (first call, second smaller call): shapes whose kernels leave split-K partials, plus one pair that
# needs none (the array is then not touched at all)
PAIRS = [
    ((1, 128, 8192, 2048), (1, 128, 2048, 2048)),     # the RMSNorm + MatMul fixture's product; tiled split-K
    ((1, 1, 2048, 8192), (1, 1, 512, 2048)),          # one-row products over row-major weights
    ((1, 4, 2048, 8192), (1, 2, 1024, 4096)),         # the few-rows kernels
    ((2, 96, 320, 4096), (1, 40, 200, 1024)),         # batched, ragged tiles
    ((1, 512, 512, 128), (1, 64, 64, 64)),            # no partials needed
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_noalloc_matmul_matches_workspace_matmul_twice_in_a_row(device, first, second):
    rng = np.random.default_rng(77)
    need_first = _both(device, rng, *first)
    need_second = _both(device, rng, *second)
    assert need_first <= SCRATCH_BYTES and need_second <= need_first
    if first[1] <= 128 and first[3] >= 2048:
        assert need_first > 0, "this pair is meant to exercise the scratch array"


def test_noalloc_matmul_broadcast_weights_then_smaller(device):
    rng = np.random.default_rng(78)
    _both(device, rng, 3, 64, 256, 4096, b_broadcast=True)
    _both(device, rng, 2, 16, 128, 2048, b_broadcast=True)


def test_noalloc_matmul_rejects_problems_beyond_its_array(device):
    from rmlk_amd import kernels as kk
    from rmlk_amd._lib import RmlkError
    # a split-K problem whose partials exceed the array (4 slabs of 768 x 3072 floats = 36 MiB)
    cand = [(1, 768, 3072, 4096), (1, 896, 3072, 8192)]
    big = [c for c in cand if kk.matmul_workspace_size(*c) > SCRATCH_BYTES]
    assert big, [kk.matmul_workspace_size(*c) for c in cand]
    batch, m, n, k = big[0]
    # the call must fail before it touches its operands: tiny stand-in buffers are enough
    t = torch.zeros(16, device=device)
    with pytest.raises(RmlkError) as err:
        kk.matmul_noalloc(t, t, t, batch, m, n, k, k, n, n, m * k, n * k, m * n)
    assert err.value.status == -8
    assert "scratch" in err.value.message
    # and the entry point still works afterwards
    rng = np.random.default_rng(79)
    _both(device, rng, 1, 128, 1024, 2048)

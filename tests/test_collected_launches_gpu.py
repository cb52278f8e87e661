"""Operators over tiny tensors collected into one launch (rmlk_hip_batch_begin / _end).

The reference launches one kernel per operator; a collected operator must give the BITS of its own
kernel (it runs the same element functors), keep its place in the order of effects on the stream,
and stay correct when the batch is full, recorded into a graph, or refused (too large, too many
dims, a type the batch does not take): then the operator's own kernel runs, behind whatever was
collected before it.
"""
import numpy as np
import pytest

from helpers import assert_exact, bcast_strides, to_dev, to_np

pytestmark = pytest.mark.gpu


def _k():
    from rmlk_amd import kernels
    return kernels


def _rand(rng, shape, dtype):
    if np.dtype(dtype).kind == "f":
        return (rng.standard_normal(shape) * 3).astype(dtype)
    return rng.integers(-50, 50, size=shape).astype(dtype)


SHAPES = [
    ((3, 1, 5), (1, 4, 5)),              # both sides broadcast
    ((1,), (7,)),                        # scalar against a row
    ((2, 3, 4, 5, 1, 2), (2, 3, 4, 5, 1, 2)),   # six dims that merge into one
    ((2, 1, 3, 1, 2, 1, 3), (1, 2, 1, 3, 1, 2, 1)),   # seven dims that do not merge: the operator's own kernel
    ((16, 64), (16, 1)),                 # 1024 elements: the largest collected
    ((17, 64), (1, 64)),                 # one row more: not collected
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
@pytest.mark.parametrize("sa,sb", SHAPES)
def test_collected_binary_ops_give_their_kernels_bits(device, dtype, sa, sb):
    import torch
    kk = _k()
    rng = np.random.default_rng(len(sa) * 13 + sa[0])
    out_shape = list(np.broadcast_shapes(sa, sb))
    a_np, b_np = _rand(rng, sa, dtype), _rand(rng, sb, dtype)
    b_np[b_np == 0] = 3                   # (integer division by zero is defined, but keep Div interesting)
    a, b = to_dev(a_np, device), to_dev(b_np, device)
    ast, bst = bcast_strides(sa, out_shape), bcast_strides(sb, out_shape)
    n = int(np.prod(out_shape))
    ops = [kk.ADD, kk.SUB, kk.MUL, kk.DIV, kk.EQUAL, kk.GREATER]
    alone, together = [], []
    for op in ops:
        odt = torch.bool if op in (kk.EQUAL, kk.GREATER) else a.dtype
        alone.append(torch.zeros(n, dtype=odt, device=device))
        together.append(torch.zeros(n, dtype=odt, device=device))
        kk.binary(op, a, b, alone[-1], out_shape, ast, bst)
    with kk.collected_launches():
        for op, out in zip(ops, together):
            kk.binary(op, a, b, out, out_shape, ast, bst)
    for x, y in zip(alone, together):
        assert_exact(to_np(y), to_np(x))


def test_collected_maps_casts_selects_and_copies(device):
    import torch
    kk = _k()
    rng = np.random.default_rng(3)
    x32 = to_dev((rng.standard_normal(1000) * 4).astype(np.float32), device)
    x64 = to_dev(rng.standard_normal(77).astype(np.float64), device)
    ints = to_dev(rng.integers(-5, 5, size=300).astype(np.int64), device)
    pos = to_dev(np.abs(rng.standard_normal(1000)).astype(np.float32), device)
    cond = to_dev(rng.random((6, 1, 5)) < 0.5, device)
    wx = to_dev(rng.standard_normal((6, 4, 5)).astype(np.float32), device)
    wy = to_dev(rng.standard_normal((1, 4, 1)).astype(np.float32), device)
    ex = to_dev(rng.integers(0, 9, size=(1, 3, 1)).astype(np.int64), device)
    c1 = to_dev(rng.standard_normal((2, 3, 4)).astype(np.float32), device)
    c2 = to_dev(rng.standard_normal((2, 5, 4)).astype(np.float32), device)
    c3 = to_dev(np.zeros((2, 0, 4), np.float32), device)

    def run(outs):
        i = iter(outs)
        for op in (kk.SQRT, kk.NEG, kk.SIN, kk.COS, kk.SIGMOID):
            kk.unary(op, pos if op == kk.SQRT else x32, next(i))
        kk.unary(kk.COS, x64, next(i))
        kk.unary(kk.NEG, ints, next(i))                      # integer Neg: not collected, runs in place
        for src, dst in ((x32, torch.int64), (x32, torch.int32), (x32, torch.bool), (ints, torch.float32),
                         (ints, torch.float64), (ints, torch.bool), (cond.reshape(-1), torch.int64),
                         (x32, torch.float16)):              # (to half: not collected)
            kk.cast(src, next(i))
        kk.where(wx, wy, cond, next(i), [6, 4, 5], bcast_strides((6, 4, 5), (6, 4, 5)),
                 bcast_strides((1, 4, 1), (6, 4, 5)), bcast_strides((6, 1, 5), (6, 4, 5)))
        kk.expand(ex, next(i), [1, 3, 1], [2, 4, 3, 5])
        kk.concat([c1, c2, c3], next(i), [[2, 3, 4], [2, 5, 4], [2, 0, 4]], [2, 8, 4], 1)

    def outputs():
        z = lambda n, dt: torch.zeros(n, dtype=dt, device=device)
        return ([z(1000, torch.float32) for _ in range(5)] + [z(77, torch.float64), z(300, torch.int64)] +
                [z(1000, torch.int64), z(1000, torch.int32), z(1000, torch.bool), z(300, torch.float32),
                 z(300, torch.float64), z(300, torch.bool), z(30, torch.int64), z(1000, torch.float16)] +
                [z(120, torch.float32), z(120, torch.int64), z(64, torch.float32)])

    alone, together = outputs(), outputs()
    run(alone)
    with kk.collected_launches():
        run(together)
    for x, y in zip(alone, together):
        assert_exact(to_np(y.view(torch.int16) if y.dtype == torch.float16 else y),
                     to_np(x.view(torch.int16) if x.dtype == torch.float16 else x))


def test_collected_chain_keeps_the_order_of_effects(device):
    """The set-up chain of a decode step (position -> rotary tables) as one batch: every record reads
    what the one before it wrote; a large operator in the middle and a reduction at the end read
    collected results through their own kernels; the buffer of a dead intermediate is reused."""
    import torch
    kk = _k()
    rng = np.random.default_rng(9)
    pos = to_dev(np.array([137], dtype=np.int64), device)
    inv = to_dev((1.0 / (500000.0 ** (np.arange(32) / 32.0))).astype(np.float32), device)
    big = to_dev(rng.standard_normal((128, 64)).astype(np.float32), device)

    def run():
        posf = torch.zeros(1, device=device)
        kk.cast(pos, posf)
        freqs = torch.zeros(32, device=device)
        kk.binary(kk.MUL, inv, posf, freqs, [32], [1], [0])
        emb = torch.zeros(64, device=device)
        kk.concat([freqs, freqs], emb, [[32], [32]], [64], 0)
        cos, sin = torch.zeros(64, device=device), torch.zeros(64, device=device)
        kk.unary(kk.COS, emb, cos)
        kk.unary(kk.SIN, emb, sin)
        # 8192 elements: this operator's own kernel, reading the collected cos
        scaled = torch.zeros(128, 64, device=device)
        kk.binary(kk.MUL, big, cos, scaled, [128, 64], [64, 1], [0, 1])
        # freqs is dead: overwrite it (as a buffer pool would hand it out again), then read it
        kk.binary(kk.ADD, sin, posf, freqs, [32], [1], [0])       # (the first 32 values of sin)
        total = torch.zeros(128, device=device)
        kk.reduce_mean(scaled, total, [128, 64], [1])
        return [posf, emb, cos, sin, scaled, freqs, total]

    alone = run()
    with kk.collected_launches():
        together = run()
    for x, y in zip(alone, together):
        assert_exact(to_np(y), to_np(x))
    exp = np.cos(np.concatenate([to_np(inv) * np.float32(137)] * 2).astype(np.float64)).astype(np.float32)
    np.testing.assert_allclose(to_np(together[2]), exp, rtol=1e-4, atol=1e-5)


def test_more_records_than_one_launch_holds(device):
    import torch
    kk = _k()
    x = to_dev(np.arange(100, dtype=np.int64), device)
    one = to_dev(np.array([1], dtype=np.int64), device)
    bufs = [torch.zeros(100, dtype=torch.int64, device=device) for _ in range(2)]
    with kk.collected_launches() as batch:
        kk.binary(kk.ADD, x, one, bufs[0], [100], [1], [0])
        for i in range(70):                   # three launches' worth of dependent records
            kk.binary(kk.ADD, bufs[i % 2], one, bufs[(i + 1) % 2], [100], [1], [0])
        batch.flush()
        torch.cuda.synchronize()
        assert np.array_equal(to_np(bufs[0]), np.arange(100) + 71)   # visible after a flush, batch still open
        kk.binary(kk.ADD, bufs[0], one, bufs[1], [100], [1], [0])
    assert np.array_equal(to_np(bufs[1]), np.arange(100) + 72)


def test_a_batch_recorded_into_a_graph_replays(device):
    import torch
    kk = _k()
    x = torch.arange(50, dtype=torch.float32, device=device)
    y = torch.zeros(50, device=device)
    z = torch.zeros(50, device=device)
    two = torch.full((1,), 2.0, device=device)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            with kk.collected_launches():
                kk.binary(kk.MUL, x, two, y, [50], [1], [0])
                kk.unary(kk.COS, y, z)
    for step in range(3):
        x.copy_(torch.arange(50, dtype=torch.float32, device=device) + step)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        exp_y = torch.zeros(50, device=device)
        exp_z = torch.zeros(50, device=device)
        kk.binary(kk.MUL, x, two, exp_y, [50], [1], [0])
        kk.unary(kk.COS, exp_y, exp_z)
        assert_exact(to_np(y), to_np(exp_y))
        assert_exact(to_np(z), to_np(exp_z))


def test_batch_begin_and_end_are_paired(device):
    import torch
    from rmlk_amd._lib import RmlkError, lib
    kk = _k()
    stream = torch.cuda.current_stream().cuda_stream
    assert lib().rmlk_hip_batch_end(stream) != 0          # nothing to end
    assert lib().rmlk_hip_batch_flush(stream) == 0        # nothing to send: fine
    with kk.collected_launches():
        with pytest.raises(RmlkError):
            with kk.collected_launches():
                pass
    assert lib().rmlk_hip_batch_end(stream) != 0          # the outer one has ended the batch

"""Fused kernels and the pattern-fusion pass, on the GPU.

The reference has no fused kernels: it runs one kernel per ONNX node. The bar here is therefore the
un-fused path itself — a fused kernel must give the BITS of the chain of separate kernels it
replaces (RMSNorm: the row mean is a double-precision sum taken in a different order, so a result
may differ in the last place on rare rows; the test allows 2 ulp there and requires 99.9 % of the
elements to be identical) — plus the CPU oracle at the per-op tolerance (rtol 1e-4 / atol 1e-5).
Session tests build every graph twice (fused / one kernel per node) and compare outputs."""
import numpy as np
import pytest

from helpers import assert_close, assert_exact, bcast_strides, to_dev, to_np

pytestmark = pytest.mark.gpu


def _k():
    from rmlk_amd import kernels
    return kernels


def _dense(shape):
    return bcast_strides(shape, shape)


# ---- kernel level: fused kernel vs the chain of separate kernels through the C ABI --------------

@pytest.mark.parametrize("rows,cols", [(1, 2048), (7, 64), (512, 2048), (1500, 256), (3, 8192),
                                       (2048, 1024), (5, 4)])
@pytest.mark.parametrize("recip", [False, True])
def test_rmsnorm_matches_separate_kernels(device, rows, cols, recip):
    import torch
    k = _k()
    rng = np.random.default_rng(rows * 31 + cols)
    x = to_dev(rng.standard_normal((rows, cols), dtype=np.float32) * 3, device)
    gamma = to_dev(rng.uniform(0.5, 1.5, size=(cols,)).astype(np.float32), device)
    eps = 1e-5
    # separate kernels: Pow, ReduceMean, Add, Sqrt, Div (or Div(1, .) and Mul), Mul
    two = torch.tensor([2.0], device=device)
    epst = torch.tensor([eps], dtype=torch.float32, device=device)
    one = torch.tensor([1.0], device=device)
    sq = torch.empty_like(x)
    k.binary(k.POW, x, two, sq, [rows, cols], [cols, 1], [0, 0])
    mean = torch.empty(rows, device=device)
    k.reduce_mean(sq, mean, [rows, cols], [1])
    var = torch.empty_like(mean)
    k.binary(k.ADD, mean, epst, var, [rows], [1], [0])
    r = torch.empty_like(mean)
    k.unary(k.SQRT, var, r)
    normed = torch.empty_like(x)
    if recip:
        inv = torch.empty_like(r)
        k.binary(k.DIV, one, r, inv, [rows], [0], [1])
        k.binary(k.MUL, x, inv, normed, [rows, cols], [cols, 1], [1, 0])
    else:
        k.binary(k.DIV, x, r, normed, [rows, cols], [cols, 1], [1, 0])
    exp = torch.empty_like(x)
    k.binary(k.MUL, normed, gamma, exp, [rows, cols], [cols, 1], [0, 1])
    got = torch.empty_like(x)
    k.rmsnorm(x, gamma, got, rows, cols, eps, recip)
    g, e = to_np(got), to_np(exp)
    same = np.mean(g.view(np.uint32) == e.view(np.uint32))
    assert same >= 0.999, same
    np.testing.assert_allclose(g, e, rtol=3e-7, atol=0)
    # oracle
    xn = to_np(x).astype(np.float64)
    ref = xn / np.sqrt((xn * xn).mean(-1, keepdims=True) + eps) * to_np(gamma)
    assert_close(g, ref.astype(np.float32), rtol=1e-4, atol=1e-5)


def test_rmsnorm_rejects_layouts_it_does_not_cover(device):
    import torch
    from rmlk_amd import RmlkError
    k = _k()
    x = torch.ones(2, 6, device=device)
    with pytest.raises(RmlkError):
        k.rmsnorm(x, torch.ones(6, device=device), torch.empty_like(x), 2, 6, 1e-5)


@pytest.mark.parametrize("n", [1, 3, 4, 8192, 512 * 8192, 1000003])
def test_swiglu_matches_separate_kernels(device, n):
    import torch
    k = _k()
    rng = np.random.default_rng(n)
    g = to_dev(rng.standard_normal(n, dtype=np.float32) * 4, device)
    u = to_dev(rng.standard_normal(n, dtype=np.float32), device)
    sig, silu, exp, got = (torch.empty_like(g) for _ in range(4))
    k.unary(k.SIGMOID, g, sig)
    k.binary(k.MUL, g, sig, silu, [n], [1], [1])
    k.binary(k.MUL, silu, u, exp, [n], [1], [1])
    k.swiglu(g, u, got)
    assert_exact(to_np(got), to_np(exp))
    gn = to_np(g).astype(np.float64)
    ref = gn / (1 + np.exp(-gn)) * to_np(u)
    assert_close(to_np(got), ref.astype(np.float32), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape,mask_shape,mul", [
    ([1, 32, 512, 640], [1, 1, 512, 640], False),
    ([1, 32, 1, 640], [1, 1, 1, 640], False),
    ([2, 4, 16, 128], [2, 1, 16, 128], True),
    ([2, 4, 16, 128], [128], False),
    ([3, 5000], [3, 5000], False),
    ([2, 3, 4, 8], [3, 1, 8], True),
    ([2, 3, 4, 5, 8], [1, 1, 4, 5, 8], True),
])
def test_scale_mask_softmax_matches_separate_kernels(device, shape, mask_shape, mul):
    import torch
    k = _k()
    rng = np.random.default_rng(sum(shape))
    x = to_dev(rng.standard_normal(shape, dtype=np.float32) * 5, device)
    mask_np = np.where(rng.random(mask_shape) < 0.3, -np.inf, 0.0).astype(np.float32)
    mask_np[..., 0] = 0.0   # no fully masked row
    mask = to_dev(mask_np, device)
    scale = 0.125 if mul else 8.0
    st = torch.tensor([scale], device=device)
    n = x.numel()
    scaled, masked, exp, got = (torch.empty_like(x) for _ in range(4))
    zeros = [0] * len(shape)
    k.binary(k.MUL if mul else k.DIV, x, st, scaled, shape, _dense(shape), zeros)
    ms = bcast_strides(mask_shape, shape)
    k.binary(k.ADD, scaled, mask, masked, shape, _dense(shape), ms)
    k.softmax(masked, exp, n // shape[-1], shape[-1], 1)
    ms_fused = list(ms)
    ms_fused[-1] = 1
    k.scale_mask_softmax(x, mask, got, shape, ms_fused, scale, mul)
    assert_exact(to_np(got), to_np(exp))
    xn = to_np(x).astype(np.float64)
    z = (xn * scale if mul else xn / scale) + mask_np
    z = z - z.max(-1, keepdims=True)
    ref = np.exp(z) / np.exp(z).sum(-1, keepdims=True)
    assert_close(to_np(got), ref.astype(np.float32), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("b,h,s,d,transposed", [
    (1, 32, 512, 64, True), (1, 8, 1, 64, True), (1, 8, 1, 64, False), (2, 3, 5, 8, False),
    (2, 3, 5, 6, True), (1, 2, 7, 2, False), (1, 4, 9, 128, True),
])
def test_rotary_matches_separate_kernels(device, b, h, s, d, transposed):
    import torch
    k = _k()
    rng = np.random.default_rng(b + h + s + d)
    shape = [b, h, s, d]
    half = d // 2
    if transposed:   # storage [B,S,H,D], logical x = Transpose(0,2,1,3)
        store = to_dev(rng.standard_normal((b, s, h, d), dtype=np.float32), device)
        x = torch.empty(b * h * s * d, device=device)
        k.transpose(store, x, [b, s, h, d], [0, 2, 1, 3])
        x_stride = [s * h * d, d, h * d, 1]
        src = store
    else:
        x = to_dev(rng.standard_normal(shape, dtype=np.float32), device).reshape(-1)
        x_stride = _dense(shape)
        src = x
    cos = to_dev(rng.uniform(-1, 1, size=(1, 1, s, d)).astype(np.float32), device)
    sin = to_dev(rng.uniform(-1, 1, size=(1, 1, s, d)).astype(np.float32), device)
    cs = bcast_strides([1, 1, s, d], shape)
    cs[-1] = 1
    n = b * h * s * d
    hs = [b, h, s, half]
    x1, x2, neg = (torch.empty(n // 2, device=device) for _ in range(3))
    k.slice_(x, x1, shape, [0, 0, 0, 0], [1, 1, 1, 1], hs)
    k.slice_(x, x2, shape, [0, 0, 0, half], [1, 1, 1, 1], hs)
    k.unary(k.NEG, x2, neg)
    rot, a, r, exp, got = (torch.empty(n, device=device) for _ in range(5))
    k.concat_into(neg, rot, hs, shape, 3, 0)
    k.concat_into(x1, rot, hs, shape, 3, half)
    bc = bcast_strides([1, 1, s, d], shape)
    k.binary(k.MUL, x, cos, a, shape, _dense(shape), bc)
    k.binary(k.MUL, rot, sin, r, shape, _dense(shape), bc)
    k.binary(k.ADD, a, r, exp, shape, _dense(shape), _dense(shape))
    k.rotary(src, cos, sin, got, shape, x_stride, cs, cs)
    assert_exact(to_np(got), to_np(exp))


@pytest.mark.parametrize("b,hq,hk,s,length,d", [
    (1, 32, 8, 512, 640, 64), (1, 32, 8, 1, 640, 64), (2, 4, 2, 5, 9, 8), (1, 2, 1, 3, 4, 6), (1, 3, 3, 7, 7, 2),
])
def test_head_rows_match_separate_kernels(device, b, hq, hk, s, length, d):
    """q rotated, k rotated into the key cache, v moved into the value cache in ONE launch equal the
    five separate kernels (rotary x2, transpose, ScatterND x2) bit for bit."""
    import torch
    k = _k()
    rng = np.random.default_rng(hq + s + d)
    def proj(h):   # a projection output [B,S,H,D]; its logical [B,H,S,D] strides
        return to_dev(rng.standard_normal((b, s, h, d), dtype=np.float32), device), [s * h * d, d, h * d, 1]
    q_st, q_xs = proj(hq)
    k_st, k_xs = proj(hk)
    v_st, v_xs = proj(hk)
    cos = to_dev(rng.uniform(-1, 1, size=(1, 1, s, d)).astype(np.float32), device)
    sin = to_dev(rng.uniform(-1, 1, size=(1, 1, s, d)).astype(np.float32), device)
    cache_shape = [b, hk, length, d]
    kc = rng.standard_normal(cache_shape, dtype=np.float32)
    vc = rng.standard_normal(cache_shape, dtype=np.float32)
    pos = rng.permutation(length)[:s]
    idx = np.zeros((b, hk, s, 3), np.int64)
    idx[..., 0] = np.arange(b).reshape(b, 1, 1)
    idx[..., 1] = np.arange(hk).reshape(1, hk, 1)
    idx[..., 2] = pos.reshape(1, 1, s)
    idx[0, 0, 0, 2] -= length                      # a negative index wraps
    idx_d = to_dev(idx, device)
    def table(h):
        cs = bcast_strides([1, 1, s, d], [b, h, s, d])
        cs[-1] = 1
        return cs
    # separate kernels
    q_exp = torch.empty(b * hq * s * d, device=device)
    k_rot = torch.empty(b * hk * s * d, device=device)
    v_tr = torch.empty(b * hk * s * d, device=device)
    k.rotary(q_st, cos, sin, q_exp, [b, hq, s, d], q_xs, table(hq), table(hq))
    k.rotary(k_st, cos, sin, k_rot, [b, hk, s, d], k_xs, table(hk), table(hk))
    k.transpose(v_st, v_tr, [b, s, hk, d], [0, 2, 1, 3])
    kc_exp, vc_exp = to_dev(kc, device), to_dev(vc, device)
    k.scatter_nd(idx_d, k_rot, kc_exp, cache_shape, b * hk * s, 3)
    k.scatter_nd(idx_d, v_tr, vc_exp, cache_shape, b * hk * s, 3)
    # one launch
    q_got = torch.empty_like(q_exp)
    kc_got, vc_got = to_dev(kc, device), to_dev(vc, device)
    err = torch.zeros(1, dtype=torch.int32, device=device)
    k.head_rows([
        dict(x=q_st, shape=[b, hq, s, d], x_stride=q_xs, cos=cos, sin=sin, cos_stride=table(hq),
             sin_stride=table(hq), out=q_got),
        dict(x=k_st, shape=[b, hk, s, d], x_stride=k_xs, cos=cos, sin=sin, cos_stride=table(hk),
             sin_stride=table(hk), out=kc_got, idx=idx_d, data_shape=cache_shape),
        dict(x=v_st, shape=[b, hk, s, d], x_stride=v_xs, out=vc_got, idx=idx_d, data_shape=cache_shape),
    ], err)
    assert_exact(to_np(q_got), to_np(q_exp))
    assert_exact(to_np(kc_got), to_np(kc_exp))
    assert_exact(to_np(vc_got), to_np(vc_exp))
    assert int(err.item()) == 0


@pytest.mark.parametrize("b,hq,hk,s,length,d,splits", [(1, 32, 8, 512, 640, 64, 2), (1, 32, 8, 512, 640, 64, 4),
                                                      (2, 4, 2, 7, 12, 16, 3), (1, 3, 1, 5, 9, 6, 2)])
def test_head_rows_over_the_partial_sums_of_a_joint_product(device, b, hq, hk, s, length, d, splits):
    """The rows of a joint q/k/v product read from its split-K slabs (added up in ascending order while
    they are loaded) equal the rows of the combined product: same bits as adding the slabs first."""
    import torch
    k = _k()
    rng = np.random.default_rng(hq + s + d + splits)
    total = (hq + 2 * hk) * d
    slabs = to_dev(rng.standard_normal((splits, b * s, total), dtype=np.float32), device)
    joint = slabs[0].clone()
    for z in range(1, splits):
        joint = joint + slabs[z]          # fp32 adds in ascending order, like the combine kernel
    cos = to_dev(rng.uniform(-1, 1, size=(1, 1, s, d)).astype(np.float32), device)
    sin = to_dev(rng.uniform(-1, 1, size=(1, 1, s, d)).astype(np.float32), device)
    cache_shape = [b, hk, length, d]
    kc = rng.standard_normal(cache_shape, dtype=np.float32)
    vc = rng.standard_normal(cache_shape, dtype=np.float32)
    pos = rng.permutation(length)[:s]
    idx = np.zeros((b, hk, s, 3), np.int64)
    idx[..., 0] = np.arange(b).reshape(b, 1, 1)
    idx[..., 1] = np.arange(hk).reshape(1, hk, 1)
    idx[..., 2] = pos.reshape(1, 1, s)
    idx_d = to_dev(idx, device)

    def table(h):
        cs = bcast_strides([1, 1, s, d], [b, h, s, d])
        cs[-1] = 1
        return cs
    xs = [s * total, d, total, 1]          # logical [B,H,S,D] over rows of the joint matrix

    def streams(src, q_out, k_out, v_out, **extra):
        cols = (0, hq * d, (hq + hk) * d)
        return [
            dict(x=src.reshape(-1)[cols[0]:], shape=[b, hq, s, d], x_stride=xs, cos=cos, sin=sin,
                 cos_stride=table(hq), sin_stride=table(hq), out=q_out, **extra),
            dict(x=src.reshape(-1)[cols[1]:], shape=[b, hk, s, d], x_stride=xs, cos=cos, sin=sin,
                 cos_stride=table(hk), sin_stride=table(hk), out=k_out, idx=idx_d, data_shape=cache_shape, **extra),
            dict(x=src.reshape(-1)[cols[2]:], shape=[b, hk, s, d], x_stride=xs, out=v_out, idx=idx_d,
                 data_shape=cache_shape, **extra)]
    err = torch.zeros(1, dtype=torch.int32, device=device)
    q_exp = torch.empty(b * hq * s * d, device=device)
    kc_exp, vc_exp = to_dev(kc, device), to_dev(vc, device)
    k.head_rows(streams(joint, q_exp, kc_exp, vc_exp), err)
    q_got = torch.full_like(q_exp, 3.0)
    kc_got, vc_got = to_dev(kc, device), to_dev(vc, device)
    k.head_rows(streams(slabs, q_got, kc_got, vc_got, partials=splits, partial_stride=b * s * total), err)
    assert_exact(to_np(q_got), to_np(q_exp))
    assert_exact(to_np(kc_got), to_np(kc_exp))
    assert_exact(to_np(vc_got), to_np(vc_exp))
    assert int(err.item()) == 0


def test_head_rows_flag_an_index_out_of_range_and_check_their_arguments(device):
    import torch
    from rmlk_amd import RmlkError
    k = _k()
    x = to_dev(np.ones((1, 2, 3, 4), np.float32), device)
    cache = to_dev(np.zeros((1, 2, 5, 4), np.float32), device)
    idx = np.zeros((1, 2, 3, 3), np.int64)
    idx[..., 1] = np.arange(2).reshape(1, 2, 1)
    idx[..., 2] = np.array([0, 5, 2]).reshape(1, 1, 3)     # 5 is past the end of the cache
    err = torch.zeros(1, dtype=torch.int32, device=device)
    st = dict(x=x, shape=[1, 2, 3, 4], x_stride=[24, 12, 4, 1], out=cache, idx=to_dev(idx, device),
              data_shape=[1, 2, 5, 4])
    k.head_rows([st], err)
    assert int(err.item()) == 1
    got = to_np(cache)
    assert got[0, :, [0, 2]].min() == 1.0 and got[0, :, [1, 3, 4]].max() == 0.0
    with pytest.raises(RmlkError):       # tuple size must address whole rows
        k.head_rows([dict(st, data_shape=[1, 2, 5, 8])], err)
    with pytest.raises(RmlkError):       # more streams than one launch takes
        k.head_rows([st] * 5, err)
    with pytest.raises(RmlkError):       # streams of different row lengths
        k.head_rows([st, dict(x=x, shape=[1, 2, 6, 2], x_stride=[24, 12, 2, 1], out=x)], err)
    k.head_rows([], err)                 # nothing to do


@pytest.mark.parametrize("hq,hk,d,k,length,normed", [(32, 8, 64, 2048, 640, True), (32, 8, 64, 2048, 640, False),
                                                     (6, 2, 64, 384, 40, True), (4, 4, 16, 100, 9, False),
                                                     (3, 1, 128, 520, 33, True)])
def test_one_token_projection_with_its_head_rows_in_one_launch(device, hq, hk, d, k, length, normed):
    """The q/k/v projection of one token, rotated / scattered behind it, in ONE launch equals the
    one-row product followed by the row-stream launch bit for bit."""
    import torch
    kk = _k()
    rng = np.random.default_rng(hq + d + k)
    n = (hq + 2 * hk) * d
    x = to_dev(rng.standard_normal(k, dtype=np.float32), device)
    wt = to_dev((rng.standard_normal((n, k), dtype=np.float32) * 0.05), device)
    gamma = to_dev(rng.uniform(0.5, 1.5, size=k).astype(np.float32), device) if normed else None
    cos = to_dev(rng.uniform(-1, 1, size=(1, 1, 1, d)).astype(np.float32), device)
    sin = to_dev(rng.uniform(-1, 1, size=(1, 1, 1, d)).astype(np.float32), device)
    cache_shape = [1, hk, length, d]
    kc = rng.standard_normal(cache_shape, dtype=np.float32)
    vc = rng.standard_normal(cache_shape, dtype=np.float32)
    idx = np.zeros((1, hk, 1, 3), np.int64)
    idx[0, :, 0, 1] = np.arange(hk)
    idx[0, :, 0, 2] = length - 2
    idx[0, 0, 0, 2] -= length                        # a negative index wraps
    idx_d = to_dev(idx, device)
    tab = [0, 0, 0, 1]
    # two launches
    y = torch.empty(n, device=device)
    if normed:
        kk.gemv_kmajor_normed(x, gamma, wt, y, n, k, 1e-5)
    else:
        kk.gemv_kmajor(x, wt, y, n, k)
    q_exp = torch.empty(hq * d, device=device)
    kc_exp, vc_exp = to_dev(kc, device), to_dev(vc, device)
    err = torch.zeros(1, dtype=torch.int32, device=device)
    def streams(q_out, k_out, v_out, src=None):
        def with_x(dct, first, h):
            if src is not None:
                dct.update(x=src[first:first + h * d], x_stride=[h * d, d, h * d, 1])
            return dct
        return [
            with_x(dict(shape=[1, hq, 1, d], cos=cos, sin=sin, cos_stride=tab, sin_stride=tab, out=q_out), 0, hq),
            with_x(dict(shape=[1, hk, 1, d], cos=cos, sin=sin, cos_stride=tab, sin_stride=tab, out=k_out,
                        idx=idx_d, data_shape=cache_shape), hq * d, hk),
            with_x(dict(shape=[1, hk, 1, d], out=v_out, idx=idx_d, data_shape=cache_shape), (hq + hk) * d, hk)]
    kk.head_rows(streams(q_exp, kc_exp, vc_exp, src=y), err)
    # one launch
    q_got = torch.full_like(q_exp, 9.0)
    kc_got, vc_got = to_dev(kc, device), to_dev(vc, device)
    kk.gemv_kmajor_head_rows(x, wt, k, streams(q_got, kc_got, vc_got), [0, hq * d, (hq + hk) * d],
                             gamma=gamma, eps=1e-5, err_flag=err)
    assert_exact(to_np(q_got), to_np(q_exp))
    assert_exact(to_np(kc_got), to_np(kc_exp))
    assert_exact(to_np(vc_got), to_np(vc_exp))
    assert int(err.item()) == 0
    # an index past the end of the cache: the flag, and that head's row is not written
    idx[0, hk - 1, 0, 2] = length
    kc_bad = to_dev(kc, device)
    st = streams(q_got, kc_bad, vc_got)[:2]
    st[1]["idx"] = to_dev(idx, device)
    kk.gemv_kmajor_head_rows(x, wt, k, st, [0, hq * d], gamma=gamma, eps=1e-5, err_flag=err)
    assert int(err.item()) == 1
    got = to_np(kc_bad)
    assert_exact(got[0, hk - 1], kc[0, hk - 1])
    if hk > 1:
        assert_exact(got[0, :hk - 1], to_np(kc_exp)[0, :hk - 1])


# ---- session level: the fusion pass ------------------------------------------------------------

def _run_both(graph, feeds, outputs=None):
    from rmlk_amd import runtime
    fused = runtime.Builder.from_graph(graph).build(fuse=True)
    plain = runtime.Builder.from_graph(graph).build(fuse=False)
    assert plain.fused_nodes == 0
    a, b = fused.run(feeds), plain.run(feeds)
    n = fused.fused_nodes
    ops = [d["op"] for d in fused.node_stats()] if hasattr(fused, "node_stats") else []
    fused.close()
    plain.close()
    return a, b, n, ops


def _same(a, b, loose=()):
    assert a.keys() == b.keys()
    for name in a:
        if a[name].dtype.kind == "f" and name in loose:
            # the attention MatMul may run on another kernel (other summation order) once fused
            np.testing.assert_allclose(a[name], b[name], rtol=1e-4, atol=1e-5)
        else:
            assert_exact(a[name], b[name])


def test_pass_forms_the_expected_nodes_on_the_llama_graph(device):
    from rmlk_amd import graphs
    cfg = graphs.LlamaConfig.tiny()
    graph = graphs.llama_graph(cfg, seed=4, style="scatter", max_len=24)
    rng = np.random.default_rng(0)
    s = 8
    feeds = {"input_ids": rng.integers(0, cfg.vocab, size=(1, s)),
             "position_ids": np.arange(s, dtype=np.int64).reshape(1, s)}
    for l in range(cfg.layers):
        for kv in ("key", "value"):
            feeds[f"cache.{l}.{kv}"] = np.zeros((1, cfg.kv_heads, 24, cfg.head_dim), np.float32)
    a, b, n, _ = _run_both(graph, feeds)
    # per layer: 2 RMSNorm, 2 rotary, 1 SwiGLU, 1 softmax, 2 attention MatMuls, those three merged
    # into one attention node, the q/k/v and the gate/up MatMul groups, 2 residual Adds merged into
    # the norm that follows and the o / down projections merged into those, the gate/up group
    # merged with the SwiGLU; plus the final RMSNorm and the lm-head (a MatMul with constant
    # weights gets a K-contiguous copy of them for one-row inputs); the rotated q and the two cache
    # updates of a layer (rotated k, transposed v) merged into one node of three row streams
    assert n == cfg.layers * 17 + 2
    # RMSNorm's mean may differ in the last place; everything downstream inherits that
    _same(a, b, loose=set(a.keys()))
    assert np.array_equal(np.argmax(a["logits"][0], -1), np.argmax(b["logits"][0], -1))


def test_fused_llama_concat_style_against_oracle(device):
    from oracle import graph as og
    from rmlk_amd import graphs, runtime
    cfg = graphs.LlamaConfig.tiny()
    graph = graphs.llama_graph(cfg, seed=4, style="concat")
    feeds = graphs.llama_concat_inputs(cfg, np.random.default_rng(1).integers(0, cfg.vocab, 9), None, 0)
    inst = runtime.Builder.from_graph(graph).build()
    assert inst.fused_nodes == cfg.layers * 17 + 2   # rotated q and k of a layer: one node of two row streams
    got = inst.run(feeds)
    exp = og.run_graph(graph, feeds)
    for name in exp:
        assert_close(got[name], exp[name], rtol=1e-3, atol=1e-4)
    inst.close()


def test_fused_decoder_layer_full_width(device):
    from rmlk_amd import graphs
    graph, feeds = graphs.decoder_layer_graph(seed=3, seq=96)
    a, b, n, _ = _run_both(graph, feeds)
    assert n == 16
    _same(a, b, loose={"y"})


def test_capture_and_replay_with_fused_nodes(device):
    from rmlk_amd import graphs, runtime
    graph, feeds = graphs.decoder_layer_graph(seed=3, seq=32)
    inst = runtime.Builder.from_graph(graph).build()
    eager = inst.run(feeds)["y"].copy()
    for name, arr in feeds.items():
        inst.set_input(name, arr)
    inst.execute()
    inst.capture()
    for _ in range(3):
        inst.replay()
        inst.sync()
        assert_exact(inst.output("y"), eager)
    inst.close()


def _builder():
    from rmlk_amd import runtime
    return runtime.GraphBuilder()


def _rmsnorm_nodes(g, x, gamma, out, recip=False, axis=-1, expose_mean=False):
    g.constant("two", np.array(2.0, np.float32))
    g.constant("eps", np.array(1e-5, np.float32))
    g.op("Pow", [x, "two"], ["sq"])
    g.op("ReduceMean", ["sq"], ["mean"]).attr("axes", [axis]).attr("keepdims", 1)
    g.op("Add", ["mean", "eps"], ["var"])
    g.op("Sqrt", ["var"], ["rms"])
    if recip:
        g.constant("one", np.array(1.0, np.float32))
        g.op("Div", ["one", "rms"], ["inv"])
        g.op("Mul", [x, "inv"], ["normed"])
    else:
        g.op("Div", [x, "rms"], ["normed"])
    g.op("Mul", [gamma, "normed"], [out])
    g.output(out)
    if expose_mean:
        g.output("mean")


@pytest.mark.parametrize("rows", [1, 5, 200])
def test_constant_weights_that_something_else_reads_stay_as_they_are(device, rows):
    """Fused product nodes keep their weights K-contiguous and release the row-major initializer -
    unless another node reads it, it is a graph output, or two products share it."""
    from oracle import graph as og
    k, n = 64, 128
    rng = np.random.default_rng(rows)
    g = _builder()
    g.input("x", np.float32, [1, rows, k])
    g.input("z", np.float32, [1, rows, k])
    g.constant("w_shared", rng.standard_normal((k, n), dtype=np.float32) * np.float32(0.1))   # two products
    g.constant("w_read", rng.standard_normal((k, n), dtype=np.float32) * np.float32(0.1))     # a product and an Add
    g.constant("w_out", rng.standard_normal((k, n), dtype=np.float32) * np.float32(0.1))      # a product and a graph output
    g.constant("w_q", rng.standard_normal((k, n), dtype=np.float32) * np.float32(0.1))        # a member of a group, and alone
    g.constant("w_k", rng.standard_normal((k, 2 * n), dtype=np.float32) * np.float32(0.1))
    g.constant("one", np.array(1.0, np.float32))
    g.op("MatMul", ["x", "w_shared"], ["y_shared_x"])
    g.op("MatMul", ["z", "w_shared"], ["y_shared_z"])
    g.op("MatMul", ["x", "w_read"], ["y_read"])
    g.op("Add", ["w_read", "one"], ["w_plus"])
    g.op("MatMul", ["x", "w_out"], ["y_out"])
    g.op("MatMul", ["z", "w_q"], ["y_q"])        # these two share `z` with each other and with w_shared's product
    g.op("MatMul", ["z", "w_k"], ["y_k"])
    g.op("MatMul", ["x", "w_q"], ["y_q_alone"])
    for name in ("y_shared_x", "y_shared_z", "y_read", "w_plus", "y_out", "w_out", "y_q", "y_k", "y_q_alone"):
        g.output(name)
    feeds = {"x": rng.standard_normal((1, rows, k), dtype=np.float32),
             "z": rng.standard_normal((1, rows, k), dtype=np.float32)}
    a, b, nf, ops = _run_both(g.build(), feeds)
    assert nf >= 2     # the products on x form one joint node, those on z another
    loose = {"y_shared_x", "y_shared_z", "y_read", "y_out", "y_q", "y_k", "y_q_alone"} if rows <= 8 else set()
    _same(a, b, loose=loose)     # many rows: the same sums in the same order over either form of the weights
    exp = og.run_graph(g.build(), feeds)
    for name in exp:
        assert_close(a[name], exp[name], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("rows,k,n,recip", [
    (1, 256, 96, False),       # one row: the norm is left to the product's kernel
    (1, 256, 96, True),
    (1, 64, 20000, False),     # very wide product: the norm is computed first, by its own launch
    (1, 6, 8, False),          # row length no multiple of 4: nothing is deferred
    (3, 256, 96, False),       # several rows: nothing is deferred
])
def test_norm_feeding_one_product_over_constant_weights(device, rows, k, n, recip):
    """RMSNorm -> MatMul(constant W) where only the product reads the normalised row: same bits as
    the session without fusion up to the norm's own last-place differences, and the oracle's values."""
    from oracle import graph as og
    g = _builder()
    g.input("x", np.float32, [1, rows, k])
    rng = np.random.default_rng(k + n)
    g.constant("gamma", rng.uniform(0.5, 1.5, size=(k,)).astype(np.float32))
    g.constant("w", (rng.standard_normal((k, n), dtype=np.float32) * np.float32(0.05)))
    g.constant("two", np.array(2.0, np.float32))
    g.constant("eps", np.array(1e-5, np.float32))
    g.op("Pow", ["x", "two"], ["sq"])
    g.op("ReduceMean", ["sq"], ["mean"]).attr("axes", [-1]).attr("keepdims", 1)
    g.op("Add", ["mean", "eps"], ["var"])
    g.op("Sqrt", ["var"], ["rms"])
    if recip:
        g.constant("one", np.array(1.0, np.float32))
        g.op("Div", ["one", "rms"], ["inv"])
        g.op("Mul", ["x", "inv"], ["normed"])
    else:
        g.op("Div", ["x", "rms"], ["normed"])
    g.op("Mul", ["gamma", "normed"], ["h"])
    g.op("MatMul", ["h", "w"], ["y"])
    g.output("y")
    feeds = {"x": rng.standard_normal((1, rows, k), dtype=np.float32) * np.float32(2.0)}
    a, b, nf, ops = _run_both(g.build(), feeds)
    if k % 4 == 0:
        assert nf == 2 and ops == ["rmlk.RMSNorm", "rmlk.MatMulConst"]
    else:   # no K-contiguous copy of such weights: the product stays a MatMul
        assert nf == 1 and ops == ["rmlk.RMSNorm", "MatMul"]
    _same(a, b, loose={"y"})
    exp = og.run_graph(g.build(), feeds)
    assert_close(a["y"], exp["y"], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape,recip,n_fused", [
    ([2, 5, 64], False, 1), ([2, 5, 64], True, 1),
    ([3, 6], False, 1),            # cols % 4 != 0: the node is formed, its body runs
    ([4, 16384], False, 1),        # row longer than the fused kernel holds: body runs
])
def test_rmsnorm_pattern_variants_and_fallback(device, shape, recip, n_fused):
    from oracle import graph as og
    g = _builder()
    g.input("x", np.float32, shape)
    rng = np.random.default_rng(len(shape))
    g.constant("gamma", rng.uniform(0.5, 1.5, size=(shape[-1],)).astype(np.float32))
    _rmsnorm_nodes(g, "x", "gamma", "y", recip)
    graph = g.build()
    feeds = {"x": rng.standard_normal(shape, dtype=np.float32)}
    a, b, n, _ = _run_both(graph, feeds)
    assert n == n_fused
    _same(a, b, loose={"y"})
    assert_close(a["y"], og.run_graph(graph, feeds)["y"], rtol=1e-4, atol=1e-5)


def test_rmsnorm_over_a_middle_axis_runs_the_body(device):
    g = _builder()
    g.input("x", np.float32, [2, 8, 4])
    g.constant("gamma", np.ones((4,), np.float32))
    _rmsnorm_nodes(g, "x", "gamma", "y", axis=1)
    feeds = {"x": np.random.default_rng(3).standard_normal((2, 8, 4), dtype=np.float32)}
    a, b, n, _ = _run_both(g.build(), feeds)
    assert n == 1
    _same(a, b)


def test_intermediate_that_is_a_graph_output_blocks_fusion(device):
    g = _builder()
    g.input("x", np.float32, [2, 64])
    g.constant("gamma", np.ones((64,), np.float32))
    _rmsnorm_nodes(g, "x", "gamma", "y", expose_mean=True)
    feeds = {"x": np.random.default_rng(4).standard_normal((2, 64), dtype=np.float32)}
    a, b, n, _ = _run_both(g.build(), feeds)
    assert n == 0
    _same(a, b)


def test_softmax_pattern_with_mask_broadcast_on_last_dim_runs_the_body(device):
    g = _builder()
    g.input("x", np.float32, [2, 4, 8])
    g.input("m", np.float32, [2, 4, 1])
    g.constant("c", np.array(4.0, np.float32))
    g.op("Div", ["x", "c"], ["sc"])
    g.op("Add", ["m", "sc"], ["z"])
    g.op("Softmax", ["z"], ["p"]).attr("axis", -1)
    g.output("p")
    rng = np.random.default_rng(5)
    feeds = {"x": rng.standard_normal((2, 4, 8), dtype=np.float32),
             "m": rng.standard_normal((2, 4, 1), dtype=np.float32)}
    a, b, n, _ = _run_both(g.build(), feeds)
    assert n == 1
    _same(a, b)


def test_rotary_pattern_on_rank3_runs_the_body(device):
    g = _builder()
    g.input("x", np.float32, [3, 5, 8])
    g.input("cos", np.float32, [5, 8])
    g.input("sin", np.float32, [5, 8])
    for name, v in (("z0", [0]), ("h", [4]), ("e", [8]), ("ax", [2])):
        g.constant(name, np.array(v, np.int64))
    g.op("Slice", ["x", "z0", "h", "ax"], ["x1"])
    g.op("Slice", ["x", "h", "e", "ax"], ["x2"])
    g.op("Neg", ["x2"], ["n2"])
    g.op("Concat", ["n2", "x1"], ["rot"]).attr("axis", -1)
    g.op("Mul", ["x", "cos"], ["a"])
    g.op("Mul", ["rot", "sin"], ["r"])
    g.op("Add", ["a", "r"], ["y"])
    g.output("y")
    rng = np.random.default_rng(6)
    feeds = {"x": rng.standard_normal((3, 5, 8), dtype=np.float32),
             "cos": rng.standard_normal((5, 8), dtype=np.float32),
             "sin": rng.standard_normal((5, 8), dtype=np.float32)}
    a, b, n, _ = _run_both(g.build(), feeds)
    assert n == 1
    _same(a, b)


def _rope_chain(g, x, out, tag):
    g.op("Slice", [x, "z", "h", "ax"], [tag + "x1"])
    g.op("Slice", [x, "h", "e", "ax"], [tag + "x2"])
    g.op("Neg", [tag + "x2"], [tag + "n2"])
    g.op("Concat", [tag + "n2", tag + "x1"], [tag + "rot"]).attr("axis", -1)
    g.op("Mul", [x, "cos"], [tag + "a"])
    g.op("Mul", [tag + "rot", "sin"], [tag + "r"])
    g.op("Add", [tag + "a", tag + "r"], [out])


def test_scatter_whose_updates_are_its_own_data_is_not_done_in_place(device):
    """ScatterND(d, idx, d) moves rows of an intermediate onto other rows of itself: the update in
    place that an intermediate otherwise gets would read rows it has already overwritten."""
    from oracle import graph as og
    g = _builder()
    g.input("x", np.float32, [1, 2, 64, 8])
    g.input("idx", np.int64, [1, 2, 64, 3])
    g.op("Neg", ["x"], ["d"])
    g.op("ScatterND", ["d", "idx", "d"], ["y"])
    g.output("y")
    rng = np.random.default_rng(11)
    idx = np.zeros((1, 2, 64, 3), np.int64)
    idx[..., 1] = np.arange(2).reshape(1, 2, 1)
    idx[0, 0, :, 2] = rng.permutation(64)
    idx[0, 1, :, 2] = rng.permutation(64)
    feeds = {"x": rng.standard_normal((1, 2, 64, 8), dtype=np.float32), "idx": idx}
    a, b, _, _ = _run_both(g.build(), feeds)
    exp = og.run_graph(g.build(), feeds)
    assert_exact(a["y"], exp["y"])
    assert_exact(b["y"], exp["y"])


@pytest.mark.parametrize("fuse", [True, False])
def test_scatter_destinations_copied_in_front_of_the_run(device, fuse):
    """Graph inputs that ScatterND nodes take as data (not donated) are copied by one launch in front
    of the first node: two scatters over the same input get a copy each, the input stays as fed for
    a node that reads it afterwards, and eager runs and replays of the recorded graph agree with the
    oracle bit for bit, also after the caller has changed the input."""
    from oracle import graph as og
    from rmlk_amd import runtime
    g = _builder()
    g.input("cache", np.float32, [1, 2, 16, 8])
    g.input("other", np.float32, [1, 2, 16, 8])
    g.input("rows", np.float32, [1, 2, 4, 8])
    g.input("idx_a", np.int64, [1, 2, 4, 3])
    g.input("idx_b", np.int64, [1, 2, 4, 3])
    g.op("Neg", ["rows"], ["neg_rows"])
    g.op("ScatterND", ["cache", "idx_a", "rows"], ["a"])
    g.op("ScatterND", ["cache", "idx_b", "neg_rows"], ["b"])
    g.op("ScatterND", ["other", "idx_a", "neg_rows"], ["c"])
    g.op("Add", ["cache", "other"], ["after"])
    for o in ("a", "b", "c", "after"):
        g.output(o)
    graph = g.build()
    rng = np.random.default_rng(5)

    def feeds_of(seed):
        r = np.random.default_rng(seed)
        f = {"cache": r.standard_normal((1, 2, 16, 8), dtype=np.float32),
             "other": r.standard_normal((1, 2, 16, 8), dtype=np.float32),
             "rows": r.standard_normal((1, 2, 4, 8), dtype=np.float32)}
        for name in ("idx_a", "idx_b"):
            idx = np.zeros((1, 2, 4, 3), np.int64)
            idx[..., 1] = np.arange(2).reshape(1, 2, 1)
            idx[0, 0, :, 2] = r.permutation(16)[:4]
            idx[0, 1, :, 2] = r.permutation(16)[:4]
            f[name] = idx
        return f

    sess = runtime.Builder.from_graph(graph).build(fuse=fuse)
    for seed in (1, 2):
        feeds = feeds_of(seed)
        got = sess.run(feeds)
        exp = og.run_graph(graph, feeds)
        for name in exp:
            assert_exact(got[name], exp[name])
    sess.capture()
    for seed in (3, 4, 5):
        feeds = feeds_of(seed)
        for name, arr in feeds.items():
            sess.set_input(name, arr)
        sess.replay()
        sess.sync()
        exp = og.run_graph(graph, feeds)
        for name in exp:
            assert_exact(sess.output(name), exp[name])
    sess.close()


@pytest.mark.parametrize("fuse", [True, False])
def test_kernel_error_is_reported_once_and_the_session_goes_on(device, fuse):
    """An index out of range makes the run (or the replay of the recorded graph) that holds it fail
    with "kernel failed" (ref: KernelFailed{code}, backend/scatter_nd.rs:198-203); the runs and
    replays after it, over good indices, succeed: the kernels' error flag is put back when it has
    been reported, not cleared by every run."""
    from rmlk_amd import runtime
    g = _builder()
    g.input("table", np.float32, [40, 4])
    g.input("rows", np.int64, [3])
    g.op("Gather", ["table", "rows"], ["picked"]).attr("axis", 0)
    g.op("Neg", ["picked"], ["y"])
    g.output("y")
    sess = runtime.Builder.from_graph(g.build()).build(fuse=fuse)
    table = np.arange(160, dtype=np.float32).reshape(40, 4)
    good, bad = np.array([39, 0, 3], np.int64), np.array([1, 40, 2], np.int64)
    assert_exact(sess.run({"table": table, "rows": good})["y"], -table[good])
    with pytest.raises(Exception, match="kernel failed"):
        sess.run({"table": table, "rows": bad})
    assert_exact(sess.run({"table": table, "rows": good})["y"], -table[good])
    sess.capture()
    for rows in (good, bad, good[::-1].copy(), bad, good):
        sess.set_input("rows", rows)
        if rows is bad:
            with pytest.raises(Exception, match="kernel failed"):
                sess.replay()
        else:
            sess.replay()
            sess.sync()
            assert_exact(sess.output("y"), -table[rows])
    # replays enqueued without a wait in between: the failure of the first is still reported when the
    # caller checks, once; the second ran over good indices and its result stands
    sess.set_input("rows", bad)
    sess.replay_enqueue()
    sess.set_input("rows", good)
    sess.replay_enqueue()
    with pytest.raises(Exception, match="kernel failed"):
        sess.check()
    sess.check()
    assert_exact(sess.output("y"), -table[good])
    for rows in (good[::-1].copy(), good):
        sess.set_input("rows", rows)
        sess.replay_enqueue()
    sess.check()
    assert_exact(sess.output("y"), -table[good])
    sess.close()


@pytest.mark.parametrize("s,early_reader", [(5, False), (1, False), (5, True)])
def test_rows_behind_the_projections_become_one_node(device, s, early_reader):
    """Rotary(q), Rotary(k) -> ScatterND and Transpose(v) -> ScatterND merge into one rmlk.HeadRows
    node with the bits of the separate kernels; a node that reads the rotated q before the cache
    updates keeps q out of the group."""
    hq, hk, d, length = 4, 2, 8, 11
    g = _builder()
    g.input("q_in", np.float32, [1, s, hq * d])
    g.input("k_in", np.float32, [1, s, hk * d])
    g.input("v_in", np.float32, [1, s, hk * d])
    g.input("cos", np.float32, [1, 1, s, d])
    g.input("sin", np.float32, [1, 1, s, d])
    g.input("cache_k", np.float32, [1, hk, length, d])
    g.input("cache_v", np.float32, [1, hk, length, d])
    g.input("idx", np.int64, [1, hk, s, 3])
    for name, val in (("z", [0]), ("h", [d // 2]), ("e", [d]), ("ax", [3]),
                      ("q_shape", [1, -1, hq, d]), ("kv_shape", [1, -1, hk, d])):
        g.constant(name, np.array(val, np.int64))
    for t, shp in (("q", "q_shape"), ("k", "kv_shape"), ("v", "kv_shape")):
        g.op("Reshape", [t + "_in", shp], [t + "_r"])
        g.op("Transpose", [t + "_r"], [t + "_t"]).attr("perm", [0, 2, 1, 3])
    _rope_chain(g, "q_t", "q_rot", "q.")
    if early_reader:
        g.op("Neg", ["q_rot"], ["q_neg"])
        g.output("q_neg")
    _rope_chain(g, "k_t", "k_rot", "k.")
    g.op("ScatterND", ["cache_k", "idx", "k_rot"], ["k_out"])
    g.op("ScatterND", ["cache_v", "idx", "v_t"], ["v_out"])
    for o in ("q_rot", "k_out", "v_out"):
        g.output(o)
    rng = np.random.default_rng(s)
    idx = np.zeros((1, hk, s, 3), np.int64)
    idx[..., 1] = np.arange(hk).reshape(1, hk, 1)
    idx[..., 2] = rng.permutation(length)[:s].reshape(1, 1, s)
    feeds = {"idx": idx}
    for name, shape in (("q_in", (1, s, hq * d)), ("k_in", (1, s, hk * d)), ("v_in", (1, s, hk * d)),
                        ("cos", (1, 1, s, d)), ("sin", (1, 1, s, d)),
                        ("cache_k", (1, hk, length, d)), ("cache_v", (1, hk, length, d))):
        feeds[name] = rng.standard_normal(shape, dtype=np.float32)
    a, b, n, ops = _run_both(g.build(), feeds)
    assert n == 3                       # two rotary chains, one group of streams
    assert ops.count("rmlk.HeadRows") == 1 and "ScatterND" not in ops
    assert ops.count("rmlk.Rotary") == (1 if early_reader else 0)
    _same(a, b)
    from oracle import graph as og
    exp = og.run_graph(g.build(), feeds)
    for name in exp:
        assert_close(a[name], exp[name], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("b,g,rep,s,l,d", [(1, 8, 4, 512, 640, 64), (1, 8, 4, 1, 640, 64),
                                            (2, 2, 3, 5, 7, 8), (1, 4, 1, 6, 9, 16),
                                            (1, 1, 1, 1, 33, 8)])
def test_attention_matmuls_read_the_cache_in_place(device, b, g, rep, s, l, d):
    """scores = q . K^T and ctx = p . V with the grouped-query repeat (Unsqueeze, Expand, Reshape)
    and the K transpose folded into GEMM strides; against the one-kernel-per-node session (fp32
    tolerance: the strided GEMM may pick another tile / GEMV kernel than the separate MatMul) and
    the oracle."""
    from oracle import graph as og
    h = g * rep
    gb = _builder()
    gb.input("q", np.float32, [b, h, s, d])
    gb.input("p", np.float32, [b, h, s, l])
    gb.input("k", np.float32, [b, g, l, d])
    gb.input("v", np.float32, [b, g, l, d])
    gb.constant("ax", np.array([2], np.int64))
    gb.constant("eshape", np.array([1, g, rep, 1, 1], np.int64))
    gb.constant("rshape", np.array([b, h, -1, d], np.int64))
    for t in ("k", "v"):
        if rep > 1:
            gb.op("Unsqueeze", [t, "ax"], [t + "u"])
            gb.op("Expand", [t + "u", "eshape"], [t + "e"])
            gb.op("Reshape", [t + "e", "rshape"], [t + "x"])
        else:
            gb.op("Neg", [t], [t + "n"])
            gb.op("Neg", [t + "n"], [t + "x"])
    gb.op("Transpose", ["kx"], ["kt"]).attr("perm", [0, 1, 3, 2])
    gb.op("MatMul", ["q", "kt"], ["scores"])
    gb.op("MatMul", ["p", "vx"], ["ctx"])
    gb.output("scores")
    gb.output("ctx")
    graph = gb.build()
    rng = np.random.default_rng(b + g + rep + s + l + d)
    feeds = {"q": rng.standard_normal((b, h, s, d), dtype=np.float32),
             "p": rng.random((b, h, s, l), dtype=np.float32),
             "k": rng.standard_normal((b, g, l, d), dtype=np.float32),
             "v": rng.standard_normal((b, g, l, d), dtype=np.float32)}
    a_, b_, n, _ = _run_both(graph, feeds)
    assert n == (2 if rep > 1 else 1)
    exp = og.run_graph(graph, feeds)
    for name in ("scores", "ctx"):
        assert_close(a_[name], b_[name], rtol=1e-4, atol=1e-4)
        assert_close(a_[name], exp[name], rtol=1e-4, atol=1e-4)


def test_attn_matmul_with_unexpected_expand_runs_the_body(device):
    """Expand that also grows the batch dim: the pattern is formed, the run-time check refuses it."""
    gb = _builder()
    gb.input("q", np.float32, [2, 4, 3, 8])
    gb.input("k", np.float32, [1, 2, 5, 8])
    gb.constant("ax", np.array([2], np.int64))
    gb.constant("eshape", np.array([2, 2, 2, 1, 1], np.int64))
    gb.constant("rshape", np.array([2, 4, 5, 8], np.int64))
    gb.op("Unsqueeze", ["k", "ax"], ["ku"])
    gb.op("Expand", ["ku", "eshape"], ["ke"])
    gb.op("Reshape", ["ke", "rshape"], ["kx"])
    gb.op("Transpose", ["kx"], ["kt"]).attr("perm", [0, 1, 3, 2])
    gb.op("MatMul", ["q", "kt"], ["scores"])
    gb.output("scores")
    rng = np.random.default_rng(9)
    feeds = {"q": rng.standard_normal((2, 4, 3, 8), dtype=np.float32),
             "k": rng.standard_normal((1, 2, 5, 8), dtype=np.float32)}
    a_, b_, n, _ = _run_both(gb.build(), feeds)
    assert n == 1
    _same(a_, b_)


def test_user_graph_cannot_name_internal_ops(device):
    from rmlk_amd import runtime
    g = _builder()
    g.input("x", np.float32, [4])
    g.op("rmlk.SwiGLU", ["x", "x"], ["y"])
    g.output("y")
    with pytest.raises(Exception, match="unsupported operator"):
        runtime.Builder.from_graph(g.build()).build()


@pytest.mark.parametrize("rows", [1, 3, 40])
def test_matmul_group_hands_out_the_separate_products(device, rows):
    """Three MatMuls on one input with constant weights become one node; one input row takes a
    single launch over the joint weight matrix (results are views of one row), more rows one GEMM
    per member on its column block."""
    from oracle import graph as og
    gb = _builder()
    gb.input("x", np.float32, [1, 0, 96])
    rng = np.random.default_rng(rows)
    for name, n in (("wq", 64), ("wk", 32), ("wv", 32)):
        gb.constant(name, (rng.standard_normal((96, n)) * 0.1).astype(np.float32))
    gb.op("MatMul", ["x", "wq"], ["q"])
    gb.op("Neg", ["q"], ["qn"])               # a consumer between the members
    gb.op("MatMul", ["x", "wk"], ["k"])
    gb.op("MatMul", ["x", "wv"], ["v"])
    gb.op("Add", ["k", "v"], ["kv"])
    for o in ("qn", "k", "v", "kv"):
        gb.output(o)
    graph = gb.build()
    feeds = {"x": rng.standard_normal((1, rows, 96), dtype=np.float32)}
    a, b, n, _ = _run_both(graph, feeds)
    assert n == 1
    exp = og.run_graph(graph, feeds)
    for name in a:
        assert a[name].shape == b[name].shape == exp[name].shape
        assert_close(a[name], b[name], rtol=1e-4, atol=1e-5)
        assert_close(a[name], exp[name], rtol=1e-4, atol=1e-5)


def test_matmul_group_keeps_a_weight_that_something_else_reads(device):
    gb = _builder()
    gb.input("x", np.float32, [2, 8])
    rng = np.random.default_rng(1)
    gb.constant("w1", rng.standard_normal((8, 8)).astype(np.float32))
    gb.constant("w2", rng.standard_normal((8, 4)).astype(np.float32))
    gb.op("MatMul", ["x", "w1"], ["a"])
    gb.op("MatMul", ["x", "w2"], ["b"])
    gb.op("MatMul", ["a", "w1"], ["c"])       # w1 again, on another input
    for o in ("a", "b", "c"):
        gb.output(o)
    feeds = {"x": rng.standard_normal((2, 8), dtype=np.float32)}
    a, b, n, _ = _run_both(gb.build(), feeds)
    assert n == 2      # the group, and the third product (constant weights) on its own
    for name in a:
        assert_close(a[name], b[name], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape", [[1, 1, 2048], [3, 40, 64], [2, 6]])
def test_residual_add_merges_into_the_norm_and_stays_an_output(device, shape):
    """h = a + b feeds an RMSNorm and is read again later (the residual stream): one node with two
    outputs; [2, 6] (cols % 4 != 0) runs the body."""
    from oracle import graph as og
    gb = _builder()
    gb.input("a", np.float32, shape)
    gb.input("b", np.float32, shape)
    rng = np.random.default_rng(len(shape) + shape[-1])
    gb.constant("gamma", rng.uniform(0.5, 1.5, size=(shape[-1],)).astype(np.float32))
    gb.op("Add", ["a", "b"], ["h"])
    _rmsnorm_nodes(gb, "h", "gamma", "y")
    gb.op("Mul", ["h", "y"], ["z"])
    gb.output("z")
    gb.output("h")
    graph = gb.build()
    feeds = {"a": rng.standard_normal(shape, dtype=np.float32),
             "b": rng.standard_normal(shape, dtype=np.float32)}
    a, b, n, _ = _run_both(graph, feeds)
    assert n == 2          # the RMSNorm chain, then the Add merged into it
    assert_exact(a["h"], b["h"])
    _same(a, b, loose={"y", "z"})
    exp = og.run_graph(graph, feeds)
    for name in a:
        assert_close(a[name], exp[name], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("rows,cols", [(1, 2048), (512, 2048), (1500, 256), (5, 4)])
def test_add_rmsnorm_kernel_matches_separate_kernels(device, rows, cols):
    import torch
    k = _k()
    rng = np.random.default_rng(rows + cols)
    a = to_dev(rng.standard_normal((rows, cols), dtype=np.float32), device)
    b = to_dev(rng.standard_normal((rows, cols), dtype=np.float32), device)
    gamma = to_dev(rng.uniform(0.5, 1.5, size=(cols,)).astype(np.float32), device)
    h = torch.empty_like(a)
    k.binary(k.ADD, a, b, h, [rows, cols], [cols, 1], [cols, 1])
    exp = torch.empty_like(a)
    k.rmsnorm(h, gamma, exp, rows, cols, 1e-5)
    got_h, got = torch.empty_like(a), torch.empty_like(a)
    k.add_rmsnorm(a, b, gamma, got_h, got, rows, cols, 1e-5)
    assert_exact(to_np(got_h), to_np(h))
    assert_exact(to_np(got), to_np(exp))


@pytest.mark.parametrize("rows", [1, 5, 256, 300])
def test_products_leave_their_combine_to_the_consumer(device, rows):
    """[gate | up] -> SwiGLU: with one input row the GEMV's split-K slabs are added up inside the
    SwiGLU kernel. o projection -> residual Add -> RMSNorm: with many rows the GEMM's split-K slabs
    are added up inside the norm kernel. Other row counts run the bodies."""
    from oracle import graph as og
    hid, ffn = 256, 512
    gb = _builder()
    gb.input("x", np.float32, [1, 0, hid])
    gb.input("res", np.float32, [1, 0, hid])
    rng = np.random.default_rng(rows)
    for name, shape in (("wo", (hid, hid)), ("wg", (hid, ffn)), ("wu", (hid, ffn)), ("wd", (ffn, hid))):
        gb.constant(name, (rng.standard_normal(shape) * 0.05).astype(np.float32))
    gb.constant("gamma", rng.uniform(0.5, 1.5, size=(hid,)).astype(np.float32))
    gb.op("MatMul", ["x", "wo"], ["o"])
    gb.op("Add", ["res", "o"], ["h"])
    _rmsnorm_nodes(gb, "h", "gamma", "hn")
    gb.op("MatMul", ["hn", "wg"], ["g"])
    gb.op("MatMul", ["hn", "wu"], ["u"])
    gb.op("Sigmoid", ["g"], ["sg"])
    gb.op("Mul", ["g", "sg"], ["silu"])
    gb.op("Mul", ["silu", "u"], ["act"])
    gb.op("MatMul", ["act", "wd"], ["d"])
    gb.op("Add", ["h", "d"], ["out"])
    gb.output("out")
    gb.output("h")
    graph = gb.build()
    feeds = {"x": rng.standard_normal((1, rows, hid), dtype=np.float32),
             "res": rng.standard_normal((1, rows, hid), dtype=np.float32)}
    a, b, n, _ = _run_both(graph, feeds)
    # RMSNorm, SwiGLU, AddRMSNorm, gate/up group, group + SwiGLU merge, o projection + AddRMSNorm
    # merge, the down projection (constant weights, K-contiguous copy for one row)
    assert n == 7
    exp = og.run_graph(graph, feeds)
    for name in a:
        assert_close(a[name], b[name], rtol=1e-4, atol=1e-5)
        assert_close(a[name], exp[name], rtol=1e-4, atol=1e-5)


# ---- products that share their first operand: one launch over the joint weight matrix -----------

@pytest.mark.parametrize("m,k,widths", [
    (512, 2048, [2048, 512, 512]),      # q/k/v of the 1B shape: split-K, blocks meet in the combine
    (2048, 256, [1024, 256, 256]),      # enough tiles: the GEMM's own tiles write to the members
    (256, 512, [128, 128]),
    (512, 2048, [2048, 320, 512]),      # a boundary inside a tile: members one by one
    (40, 96, [64, 32, 32]),             # ragged rows: members one by one
    (5, 256, [128, 64]),                # skinny
    (128, 64, [256, 0, 128, 128]),      # an empty member
])
def test_grouped_matmul_matches_separate_products(device, m, k, widths):
    import torch
    kk = _k()
    rng = np.random.default_rng(m + k + len(widths))
    a_np = rng.standard_normal((m, k), dtype=np.float32)
    b_np = rng.standard_normal((k, sum(widths)), dtype=np.float32) * np.float32(0.02)
    a, b = to_dev(a_np, device), to_dev(b_np, device)
    outs = [torch.full((m, w), float("nan"), device=device) for w in widths]
    kk.matmul_grouped(a, b, outs, m, k, widths)
    off = 0
    for w, got in zip(widths, outs):
        if w:
            sep = torch.empty(m, w, device=device)
            kk.matmul(a, b[:, off:off + w].contiguous(), sep, 1, m, w, k, k, w, w, 0, 0, 0)
            assert_close(to_np(got), to_np(sep), rtol=1e-4, atol=1e-5)
            exp = a_np.astype(np.float64) @ b_np[:, off:off + w].astype(np.float64)
            assert_close(to_np(got), exp.astype(np.float32), rtol=1e-4, atol=1e-5)
        off += w
    # the same over the K-contiguous form of the joint matrix: the members' rows instead of columns
    if k % 4 == 0:
        bt = to_dev(np.ascontiguousarray(b_np.T), device)
        outs_t = [torch.full((m, w), float("nan"), device=device) for w in widths]
        kk.matmul_grouped(a, bt, outs_t, m, k, widths, trans_b=True)
        off = 0
        for w, got_t, got in zip(widths, outs_t, outs):
            if w:
                sep = torch.empty(m, w, device=device)
                kk.matmul(a, bt[off:off + w], sep, 1, m, w, k, k, k, w, 0, 0, 0, trans_b=True)
                assert_close(to_np(got_t), to_np(sep), rtol=1e-4, atol=1e-5)
                if m > 8:   # the tiled kernels add up in the same order for both forms of B
                    assert_exact(to_np(got_t), to_np(got))
                else:
                    assert_close(to_np(got_t), to_np(got), rtol=1e-4, atol=1e-5)
            off += w


def test_grouped_matmul_argument_checks(device):
    import torch
    from rmlk_amd import RmlkError
    kk = _k()
    a = torch.zeros(128, 64, device=device)
    b = torch.zeros(64, 256, device=device)
    outs = [torch.zeros(128, 64, device=device) for _ in range(5)]
    with pytest.raises(RmlkError):
        kk.matmul_grouped(a, b, outs, 128, 64, [64] * 5)       # more members than the entry takes
    with pytest.raises(RmlkError):
        kk.matmul_grouped(a, b, outs[:2], 128, 64, [64, -1])


@pytest.mark.parametrize("m,n,k,gate_first", [(512, 8192, 2048, True), (256, 8192, 64, False),
                                              (2048, 1024, 512, True), (500, 8192, 256, True),
                                              (129, 8192, 128, False)])
def test_matmul_swiglu_matches_separate_kernels(device, m, n, k, gate_first):
    import torch
    kk = _k()
    rng = np.random.default_rng(m + n + k)
    a_np = rng.standard_normal((m, k), dtype=np.float32)
    b_np = rng.standard_normal((k, 2 * n), dtype=np.float32) * np.float32(0.02)
    a, b = to_dev(a_np, device), to_dev(b_np, device)
    go, uo = (0, n) if gate_first else (n, 0)
    got = torch.full((m, n), float("nan"), device=device)
    kk.matmul_swiglu(a, b, got, m, n, k, 2 * n, go, uo)
    gate, up = torch.empty(m, n, device=device), torch.empty(m, n, device=device)
    kk.matmul(a, b[:, go:go + n].contiguous(), gate, 1, m, n, k, k, n, n, 0, 0, 0)
    kk.matmul(a, b[:, uo:uo + n].contiguous(), up, 1, m, n, k, k, n, n, 0, 0, 0)
    sep = torch.empty(m, n, device=device)
    kk.swiglu(gate, up, sep)
    assert_close(to_np(got), to_np(sep), rtol=1e-4, atol=1e-5)
    g64 = a_np.astype(np.float64) @ b_np[:, go:go + n].astype(np.float64)
    u64 = a_np.astype(np.float64) @ b_np[:, uo:uo + n].astype(np.float64)
    exp = g64 / (1.0 + np.exp(-g64)) * u64
    assert_close(to_np(got), exp.astype(np.float32), rtol=1e-4, atol=1e-5)
    # K-contiguous weights ([2n, k], gate and up rows): the same sums in the same order
    bt = to_dev(np.ascontiguousarray(b_np.T), device)
    got_t = torch.full((m, n), float("nan"), device=device)
    kk.matmul_swiglu(a, bt, got_t, m, n, k, k, go, uo, trans_b=True)
    assert_exact(to_np(got_t), to_np(got))


@pytest.mark.parametrize("m,n,k", [(64, 8192, 256), (512, 8200, 256), (512, 128, 256), (512, 8192, 48),
                                   (8, 32768, 256)])
def test_matmul_swiglu_declines_what_it_does_not_cover(device, m, n, k):
    import torch
    from rmlk_amd import RmlkError
    kk = _k()
    a = torch.zeros(m, k, device=device)
    b = torch.zeros(k, 2 * n, device=device)
    out = torch.zeros(m, n, device=device)
    with pytest.raises(RmlkError) as e:
        kk.matmul_swiglu(a, b, out, m, n, k, 2 * n, 0, n)
    assert e.value.status == -2
    with pytest.raises(RmlkError) as e:
        kk.matmul_swiglu(a, b.t().contiguous(), out, m, n, k, k, 0, n, trans_b=True)
    assert e.value.status == -2


@pytest.mark.parametrize("rows", [128, 384])
def test_gate_up_swiglu_of_many_rows_is_one_launch(device, rows):
    """[gate | up] -> SwiGLU with whole row tiles: the session's fused node takes the GEMM with the
    activation in its epilogue; results against the one-kernel-per-node session and the oracle."""
    from oracle import graph as og
    hid, ffn = 128, 8192
    gb = _builder()
    gb.input("x", np.float32, [1, 0, hid])
    rng = np.random.default_rng(rows)
    for name in ("wg", "wu"):
        gb.constant(name, (rng.standard_normal((hid, ffn)) * 0.1).astype(np.float32))
    gb.op("MatMul", ["x", "wg"], ["g"])
    gb.op("MatMul", ["x", "wu"], ["u"])
    gb.op("Sigmoid", ["g"], ["sg"])
    gb.op("Mul", ["g", "sg"], ["silu"])
    gb.op("Mul", ["silu", "u"], ["act"])
    gb.output("act")
    graph = gb.build()
    feeds = {"x": rng.standard_normal((1, rows, hid), dtype=np.float32)}
    a, b, n, _ = _run_both(graph, feeds)
    assert n == 3      # SwiGLU, the gate/up group, their merge
    exp = og.run_graph(graph, feeds)
    assert_close(a["act"], b["act"], rtol=1e-4, atol=1e-5)
    assert_close(a["act"], exp["act"], rtol=1e-4, atol=1e-5)


# ---- attention over many query rows in one kernel -----------------------------------------------

def _attention_reference(q, k, v, mask, scale, mul):
    """float64 numpy: softmax(q k^T (*|/) scale + mask) v with KV heads repeated."""
    b, h, s, d = q.shape
    g = k.shape[1]
    rep = h // g
    kk = np.repeat(k.astype(np.float64), rep, axis=1)
    vv = np.repeat(v.astype(np.float64), rep, axis=1)
    sc = q.astype(np.float64) @ kk.transpose(0, 1, 3, 2)
    sc = sc * scale if mul else sc / scale
    sc = sc + np.broadcast_to(mask.astype(np.float64), sc.shape)
    sc = sc - sc.max(axis=-1, keepdims=True)
    p = np.exp(sc)
    p = p / p.sum(axis=-1, keepdims=True)
    return (p @ vv).astype(np.float32)


@pytest.mark.parametrize("b,g,rep,s,l,mask_shape,mul", [
    (1, 8, 4, 512, 640, (1, 1, 512, 640), False),     # the 1B prefill shape
    (2, 2, 3, 70, 132, (2, 1, 70, 132), True),        # ragged rows and keys, per-batch mask
    (1, 1, 1, 33, 4, (1, 1, 33, 4), False),           # fewer keys than one chunk
    (1, 2, 2, 64, 256, (1, 4, 64, 256), True),        # per-head mask
    (1, 3, 1, 200, 64, (1, 1, 1, 64), False),         # one mask row for every query
    # more blocks than compute units: four wavefronts per block instead of eight
    (1, 8, 4, 2048, 2064, (1, 1, 2048, 2064), False),
    (2, 8, 3, 700, 132, (2, 1, 700, 132), True),      # the same with ragged rows and keys
    (1, 8, 4, 512, 200, (1, 1, 512, 200), False),     # eight wavefronts, keys end inside a chunk of 128
])
def test_attention_matches_separate_kernels(device, b, g, rep, s, l, mask_shape, mul):
    import torch
    kk = _k()
    h, d = g * rep, 64
    rng = np.random.default_rng(b * 1000 + s + l)
    q_np = rng.standard_normal((b, h, s, d), dtype=np.float32)
    k_np = rng.standard_normal((b, g, l, d), dtype=np.float32)
    v_np = rng.standard_normal((b, g, l, d), dtype=np.float32)
    # causal-style mask with -inf above the diagonal of the last s keys, plus some finite biases
    m_np = rng.standard_normal(mask_shape, dtype=np.float32)
    qi = np.arange(mask_shape[2])[:, None] + (l - mask_shape[2])
    hidden = np.arange(l)[None, :] > np.maximum(qi, 0)
    m_np = np.where(np.broadcast_to(hidden, mask_shape), np.float32(-np.inf), m_np).astype(np.float32)
    scale = 8.0 if not mul else 0.125
    q, k, v, m = (to_dev(x, device) for x in (q_np, k_np, v_np, m_np))
    got = torch.full((b, h, s, d), float("nan"), device=device)
    full = [b, h, s, l]
    ms = bcast_strides(list(mask_shape), full)
    kk.attention(q, k, v, m, got, b, g, rep, s, l, d, ms, scale, mul)
    # the chain of separate kernels: scores per KV head (rows of its query heads), softmax, context
    sc = torch.empty(b, h, s, l, device=device)
    kk.matmul(q, k, sc, b * g, rep * s, l, d, d, d, l, rep * s * d, l * d, rep * s * l, trans_b=True)
    pr = torch.empty_like(sc)
    kk.scale_mask_softmax(sc, m, pr, full, ms, scale, mul)
    sep = torch.empty(b, h, s, d, device=device)
    kk.matmul(pr, v, sep, b * g, rep * s, d, l, l, d, d, rep * s * l, l * d, rep * s * d)
    assert_close(to_np(got), to_np(sep), rtol=1e-4, atol=1e-5)
    assert_close(to_np(got), _attention_reference(q_np, k_np, v_np, m_np, scale, mul), rtol=1e-4, atol=1e-5)
    # the same numbers written as [B, S, H, D]
    moved = torch.full((b, s, h, d), float("nan"), device=device)
    kk.attention(q, k, v, m, moved, b, g, rep, s, l, d, ms, scale, mul, out_seq_major=True)
    assert_exact(to_np(moved), to_np(got).transpose(0, 2, 1, 3))


@pytest.mark.parametrize("rise", [0.02, 0.3, 4.0])
@pytest.mark.parametrize("s,l", [(512, 640), (2048, 1024)])
def test_attention_scores_that_rise_along_the_keys(device, s, l, rise):
    """The point the exponents are taken from follows the running maximum only past a slack: scores
    that climb slowly (a few hundredths per key: the point trails the maximum for many chunks),
    steadily (it moves in every chunk) and steeply (by hundreds per chunk) all give the softmax of
    the float64 reference - to what fp32 scores allow: a score of size x carries an error of about
    x * 2^-24, which its probability inherits as a relative error."""
    import torch
    kk = _k()
    b, g, rep, d = 1, 8, 4, 64
    h = g * rep
    rng = np.random.default_rng(s + l + int(rise * 100))
    q_np = np.zeros((b, h, s, d), dtype=np.float32)
    k_np = np.zeros((b, g, l, d), dtype=np.float32)
    # q . k = 8 * rise * key index (+ noise): after the division by the scale 8 a climb of `rise` per key
    q_np[..., 0] = 8.0
    k_np[..., 0] = (rise * np.arange(l, dtype=np.float32))[None, None, :]
    q_np[..., 1:] = 0.1 * rng.standard_normal((b, h, s, d - 1), dtype=np.float32)
    k_np[..., 1:] = rng.standard_normal((b, g, l, d - 1), dtype=np.float32)
    v_np = rng.standard_normal((b, g, l, d), dtype=np.float32)
    m_np = np.zeros((1, 1, s, l), dtype=np.float32)
    qi = np.arange(s)[:, None] + (l - s) if l >= s else np.arange(s)[:, None] * l // s
    m_np[0, 0][np.arange(l)[None, :] > np.maximum(qi, 0)] = -np.inf
    q, k, v, m = (to_dev(x, device) for x in (q_np, k_np, v_np, m_np))
    ms = [0, 0, l, 1]
    want = _attention_reference(q_np, k_np, v_np, m_np, 8.0, False)
    atol = 1e-5 + 1e-6 * rise * l
    got = torch.full((b, h, s, d), float("nan"), device=device)
    kk.attention(q, k, v, m, got, b, g, rep, s, l, d, ms, 8.0)
    assert_close(to_np(got), want, rtol=1e-4, atol=atol)
    skipped = torch.full((b, h, s, d), float("nan"), device=device)
    tile_map = kk.attention_map(m, b, g, rep, s, l, d, ms)
    assert tile_map is not None
    kk.attention_mapped(q, k, v, m, skipped, tile_map, b, g, rep, s, l, d, ms, 8.0)
    assert_close(to_np(skipped), want, rtol=1e-4, atol=atol)


def _skipping_mask(kind, rng, mask_shape, l):
    """Masks with whole (64-query, 64-key) tiles hidden, in the shapes that occur: causal with a past,
    a sliding window (hidden tiles on both sides), random hidden tiles per batch and head (one query
    tile sees nothing at all), one mask row shared by every query."""
    mb, mh, ms_, _ = mask_shape
    m = (rng.standard_normal(mask_shape, dtype=np.float32) * 0.5).astype(np.float32)
    rows = np.arange(ms_)[:, None] + (l - ms_ if ms_ > 1 else 0)
    keys = np.arange(l)[None, :]
    if kind == "causal":
        hidden = np.broadcast_to(keys > rows, mask_shape)
    elif kind == "window":
        hidden = np.broadcast_to((keys > rows) | (keys < rows - 300), mask_shape)
    elif kind == "tiles":
        t = rng.random((mb, mh, (ms_ + 63) // 64, (l + 63) // 64)) < 0.6
        t[0, 0, 0, 0] = False
        t[0, 0, 1, :] = True          # a tile of queries that sees nothing: NaN rows
        t[-1, -1, 2, :] = True
        t[-1, -1, 2, 5] = False       # and one that sees a single chunk
        hidden = np.repeat(np.repeat(t, 64, axis=2), 64, axis=3)[:, :, :ms_, :l]
        # single visible keys inside otherwise hidden tiles keep those chunks on the list
        hidden = hidden.copy()
        hidden[0, 0, 200, 777 % l] = False
    else:                              # "row": chunks 2.. and 9 hidden for everyone
        hidden = np.zeros(mask_shape, dtype=bool)
        hidden[..., 128:448] = True
        hidden[..., 576:640] = True
    return np.where(hidden, np.float32(-np.inf), m).astype(np.float32)


@pytest.mark.parametrize("b,g,rep,s,l,mask_shape,kind,skips", [
    (1, 8, 4, 2048, 2048, (1, 1, 2048, 2048), "causal", True),    # the 2048-token prefill
    (1, 8, 4, 2048, 2064, (1, 1, 2048, 2064), "causal", True),    # with a past; keys end inside a chunk
    (1, 8, 4, 1024, 1024, (1, 1, 1024, 1024), "window", True),
    (2, 4, 3, 1024, 1024, (2, 12, 1024, 1024), "tiles", True),    # per batch and head
    (1, 8, 4, 1024, 1024, (1, 32, 1024, 1024), "tiles", True),    # per head only
    (2, 8, 4, 512, 1024, (2, 1, 512, 1024), "tiles", True),       # per batch only
    (1, 8, 4, 2048, 704, (1, 1, 1, 704), "row", True),            # one mask row for every query
    (1, 8, 4, 512, 640, (1, 1, 512, 640), "causal", False),       # a block per compute unit and five chunks of 128
    (1, 8, 4, 512, 2048, (1, 1, 512, 2048), "causal", True),      # the same prompt in a longer cache: 16 chunks
    (1, 8, 4, 512, 2000, (1, 1, 1, 2000), "row", True),           # keys end inside a chunk of 128
    (2, 2, 2, 256, 1024, (2, 4, 256, 1024), "tiles", True),       # a few blocks, per batch and head
    (1, 1, 1, 192, 900, (1, 1, 192, 900), "window", True),        # three blocks
    (1, 8, 4, 2000, 2048, (1, 1, 2000, 2048), "causal", False),   # tiles would straddle heads
    (1, 8, 4, 2048, 128, (1, 1, 2048, 128), "causal", False),     # two chunks: nothing to gain
])
def test_attention_skipping_hidden_chunks_is_bit_identical(device, b, g, rep, s, l, mask_shape, kind, skips):
    """Chunks of keys that a tile of 64 queries cannot see (-inf for all of them) have probabilities
    that are exact zeros, so leaving them out changes no bit; rows that see nothing are NaN either way."""
    import torch
    kk = _k()
    h, d = g * rep, 64
    rng = np.random.default_rng(s * 7 + l + b)
    q, k, v = (to_dev(rng.standard_normal(sh, dtype=np.float32), device)
               for sh in ((b, h, s, d), (b, g, l, d), (b, g, l, d)))
    m_np = _skipping_mask(kind, rng, mask_shape, l)
    m = to_dev(m_np, device)
    ms = bcast_strides(list(mask_shape), [b, h, s, l])
    for seq_major in (False, True):
        shape = (b, s, h, d) if seq_major else (b, h, s, d)
        plain = torch.full(shape, 7.0, device=device)
        kk.attention(q, k, v, m, plain, b, g, rep, s, l, d, ms, 8.0, False, out_seq_major=seq_major)
        got = torch.full(shape, 9.0, device=device)
        need = kk.attention_skipping(q, k, v, m, got, b, g, rep, s, l, d, ms, 8.0, False, out_seq_major=seq_major)
        assert (need > 0) == skips
        if skips:
            mb, mh = mask_shape[0], mask_shape[1]
            # chunks of 64 keys for the kernel that has more blocks than compute units, of 128 otherwise
            keys = 64 if b * g * (rep * s // 64) > 256 else 128
            assert need == (mb * mh * (s // 64) * ((l + keys - 1) // keys) + 15) // 16 * 16 + 16   # the map and a counter
        a, e = to_np(got), to_np(plain)
        assert np.array_equal(np.isnan(a), np.isnan(e))
        assert_exact(np.nan_to_num(a, nan=0.0), np.nan_to_num(e, nan=0.0))
    if kind == "tiles":
        out = to_np(plain)   # [B, S, H, D] from the last pass
        assert np.isnan(out[0, 64:128, 0]).all() and np.isfinite(out[0, :64, 0]).all()


@pytest.mark.parametrize("b,g,rep,s,l,mask_shape,kind", [
    (1, 8, 4, 2048, 2048, (1, 1, 2048, 2048), "causal"),    # items handed out from the counter
    (1, 8, 4, 512, 640, (1, 1, 512, 640), "causal"),        # a block per compute unit, five chunks of 128
    (1, 8, 4, 2048, 128, (1, 1, 2048, 128), "causal"),      # two chunks of 64
    (2, 4, 3, 1024, 1024, (2, 12, 1024, 1024), "tiles"),    # per batch and head, tiles that see nothing
    (1, 1, 1, 192, 900, (1, 1, 192, 900), "window"),
    (1, 8, 4, 512, 256, (1, 1, 1, 256), "row"),             # two chunks of 128
])
def test_attention_over_a_shared_map_is_bit_identical(device, b, g, rep, s, l, mask_shape, kind):
    """One map of the mask, made once, serves several launches with different q, k, v (the layers of a
    model): each equals the kernel that visits every chunk bit for bit, the counter behind the map is
    zero again after every launch, and the map itself is left alone."""
    import torch
    kk = _k()
    h, d = g * rep, 64
    rng = np.random.default_rng(s + 3 * l + b)
    m = to_dev(_skipping_mask(kind, rng, mask_shape, l), device)
    ms = bcast_strides(list(mask_shape), [b, h, s, l])
    tile_map = kk.attention_map(m, b, g, rep, s, l, d, ms)
    assert tile_map is not None
    before = to_np(tile_map).copy()
    keys = 64 if b * g * (rep * s // 64) > 256 else 128
    entries = mask_shape[0] * mask_shape[1] * (s // 64) * ((l + keys - 1) // keys)   # (then padding to 16 bytes)
    assert before.size == (entries + 15) // 16 * 16 + 16
    assert before[-16:-12].view(np.int32)[0] == 0 and set(np.unique(before[:entries])) <= {0, 1}
    assert 0 < before[:entries].sum() < entries
    for layer in range(3):
        q, k, v = (to_dev(rng.standard_normal(sh, dtype=np.float32), device)
                   for sh in ((b, h, s, d), (b, g, l, d), (b, g, l, d)))
        seq_major = layer == 1
        shape = (b, s, h, d) if seq_major else (b, h, s, d)
        plain = torch.full(shape, 7.0, device=device)
        kk.attention(q, k, v, m, plain, b, g, rep, s, l, d, ms, 8.0, False, out_seq_major=seq_major)
        got = torch.full(shape, 9.0, device=device)
        kk.attention_mapped(q, k, v, m, got, tile_map, b, g, rep, s, l, d, ms, 8.0, False, out_seq_major=seq_major)
        a, e = to_np(got), to_np(plain)
        assert np.array_equal(np.isnan(a), np.isnan(e))
        assert_exact(np.nan_to_num(a, nan=0.0), np.nan_to_num(e, nan=0.0))
        assert np.array_equal(to_np(tile_map), before)


def test_attention_map_refusals(device):
    import torch
    kk = _k()
    m = torch.zeros(1, 1, 100, 256, device=device)                  # q_len not a multiple of 64
    assert kk.attention_map(m, 1, 8, 4, 100, 256, 64, [0, 0, 256, 1]) is None
    m = torch.zeros(1, 1, 512, 64, device=device)                   # a single chunk
    assert kk.attention_map(m, 1, 8, 4, 512, 64, 64, [0, 0, 64, 1]) is None
    m = torch.zeros(1, 1, 512, 640, device=device)
    q = torch.zeros(1, 32, 512, 64, device=device)
    kv = torch.zeros(1, 8, 640, 64, device=device)
    small = torch.zeros(16, dtype=torch.uint8, device=device)
    with pytest.raises(kk.RmlkError):                               # a map that is too small
        kk.attention_mapped(q, kv, kv, m, torch.empty_like(q), small, 1, 8, 4, 512, 640, 64, [0, 0, 640, 1], 8.0)


def test_attention_workspace_that_is_too_small_is_not_used(device):
    """A workspace below the size the library names is ignored (every chunk is visited): nothing is
    written to it and the result is the plain kernel's."""
    import torch
    from rmlk_amd._lib import check, lib
    from rmlk_amd.kernels import Dims
    kk = _k()
    b, g, rep, s, l, d = 1, 8, 4, 1024, 1024, 64
    rng = np.random.default_rng(5)
    q, k, v = (to_dev(rng.standard_normal(sh, dtype=np.float32), device)
               for sh in ((b, g * rep, s, d), (b, g, l, d), (b, g, l, d)))
    m = to_dev(_skipping_mask("causal", rng, (1, 1, s, l), l), device)
    ms = Dims.of([0, 0, l, 1])
    need = int(lib().rmlk_hip_attention_workspace_size(kk.FLOAT, b, g, rep, s, l, d, ms))
    assert need > 16
    exp = torch.empty(b, g * rep, s, d, device=device)
    kk.attention(q, k, v, m, exp, b, g, rep, s, l, d, [0, 0, l, 1], 8.0)
    ws = torch.full((need,), 7, dtype=torch.uint8, device=device)
    got = torch.empty_like(exp)
    stream = torch.cuda.current_stream().cuda_stream
    check(lib().rmlk_hip_attention_ws(stream, kk.FLOAT, b, g, rep, s, l, d, q.data_ptr(), k.data_ptr(),
                                      v.data_ptr(), m.data_ptr(), ms, 0, 8.0, 0, ws.data_ptr(), need - 1,
                                      got.data_ptr()), "rmlk_hip_attention_ws")
    assert_exact(to_np(got), to_np(exp))
    assert (to_np(ws) == 7).all()
    # the same for one that is large enough but not 16-byte aligned
    ws2 = torch.full((need + 16,), 7, dtype=torch.uint8, device=device)
    got2 = torch.empty_like(exp)
    check(lib().rmlk_hip_attention_ws(stream, kk.FLOAT, b, g, rep, s, l, d, q.data_ptr(), k.data_ptr(),
                                      v.data_ptr(), m.data_ptr(), ms, 0, 8.0, 0, ws2.data_ptr() + 4, need,
                                      got2.data_ptr()), "rmlk_hip_attention_ws")
    assert_exact(to_np(got2), to_np(exp))
    assert (to_np(ws2) == 7).all()


def test_attention_few_rows_one_launch_needs_its_counters(device):
    import torch
    from rmlk_amd import RmlkError
    kk = _k()
    q = torch.zeros(1, 8, 1, 64, device=device)
    k = torch.zeros(1, 2, 64, 64, device=device)
    m = torch.zeros(1, 64, device=device)

    with pytest.raises(RmlkError):
        kk.attention_few_rows_one_launch(q, k, k, m, torch.zeros_like(q), None, 1, 2, 4, 1, 64, 64,
                                         [0, 0, 0, 1], 8.0)


def test_attention_skipped_chunks_do_not_read_their_keys(device):
    """What the skipped chunks hold never reaches the output: NaN in K and V rows no query of a tile
    sees leaves that tile finite (the kernel without the map gives 0 * NaN there)."""
    import torch
    kk = _k()
    b, g, rep, s, l, d = 1, 8, 4, 1024, 1024, 64
    rng = np.random.default_rng(11)
    q_np, k_np, v_np = (rng.standard_normal(sh, dtype=np.float32) for sh in ((b, g * rep, s, d), (b, g, l, d), (b, g, l, d)))
    m_np = _skipping_mask("causal", rng, (1, 1, s, l), l)
    k_bad, v_bad = k_np.copy(), v_np.copy()
    k_bad[:, :, 512:] = np.nan
    v_bad[:, :, 512:] = np.nan
    m = to_dev(m_np, device)
    got = torch.empty(b, g * rep, s, d, device=device)
    need = kk.attention_skipping(to_dev(q_np, device), to_dev(k_bad, device), to_dev(v_bad, device), m, got,
                                 b, g, rep, s, l, d, [0, 0, l, 1], 8.0)
    assert need > 0
    exp = torch.empty_like(got)
    kk.attention(to_dev(q_np, device), to_dev(k_np, device), to_dev(v_np, device), m, exp, b, g, rep, s, l, d,
                 [0, 0, l, 1], 8.0)
    assert_exact(to_np(got)[:, :, :512], to_np(exp)[:, :, :512])
    assert np.isnan(to_np(got)[:, :, 512:]).all()


def test_attention_row_with_nothing_visible_is_nan_like_softmax(device):
    import torch
    kk = _k()
    b, g, rep, s, l, d = 1, 1, 1, 40, 128, 64
    rng = np.random.default_rng(3)
    q, k, v = (to_dev(rng.standard_normal(sh, dtype=np.float32), device)
               for sh in ((b, g * rep, s, d), (b, g, l, d), (b, g, l, d)))
    m_np = np.zeros((1, 1, s, l), dtype=np.float32)
    m_np[0, 0, 7, :] = -np.inf        # nothing visible
    m_np[0, 0, 9, :100] = -np.inf     # nothing visible in the first chunk
    m = to_dev(m_np, device)
    got = torch.empty(b, g * rep, s, d, device=device)
    kk.attention(q, k, v, m, got, b, g, rep, s, l, d, [0, 0, l, 1], 8.0)
    out = to_np(got)
    assert np.isnan(out[0, 0, 7]).all()
    assert np.isfinite(np.delete(out, 7, axis=2)).all()
    exp = _attention_reference(to_np(q), to_np(k), to_np(v), np.where(np.isinf(m_np), -1e30, m_np).astype(np.float32), 8.0, False)
    assert_close(np.delete(out, 7, axis=2), np.delete(exp, 7, axis=2), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("s,l", [(64, 128), (200, 264)])
def test_attention_with_most_negative_finite_mask_matches_separate_kernels(device, s, l):
    """Exported graphs hide keys with an additive mask of float32's most negative finite value, not
    -inf. In fp32 `score + that` is that value again, so a row with every key hidden is a uniform
    average of V in the separate Add / Softmax kernels (finite), not NaN; the one-kernel attention has
    to agree, also for rows that mix hidden and visible keys."""
    import torch
    kk = _k()
    b, g, rep, d = 1, 2, 2, 64
    h = g * rep
    rng = np.random.default_rng(s + l)
    q_np, k_np, v_np = (rng.standard_normal(sh, dtype=np.float32)
                        for sh in ((b, h, s, d), (b, g, l, d), (b, g, l, d)))
    lowest = np.finfo(np.float32).min
    m_np = np.zeros((1, 1, s, l), dtype=np.float32)
    qi = np.arange(s)[:, None] + (l - s)
    m_np[0, 0][np.arange(l)[None, :] > qi] = lowest       # causal
    m_np[0, 0, 5, :] = lowest                              # a padded row: nothing visible
    m_np[0, 0, s - 1, :] = lowest
    m_np[0, 0, 9, : l - 3] = lowest                        # visible keys only in the last chunk
    q, k, v, m = (to_dev(x, device) for x in (q_np, k_np, v_np, m_np))
    full, ms = [b, h, s, l], [0, 0, l, 1]
    got = torch.full((b, h, s, d), float("nan"), device=device)
    kk.attention(q, k, v, m, got, b, g, rep, s, l, d, ms, 8.0, False)
    sc = torch.empty(b, h, s, l, device=device)
    kk.matmul(q, k, sc, b * g, rep * s, l, d, d, d, l, rep * s * d, l * d, rep * s * l, trans_b=True)
    pr = torch.empty_like(sc)
    kk.scale_mask_softmax(sc, m, pr, full, ms, 8.0, False)
    sep = torch.empty(b, h, s, d, device=device)
    kk.matmul(pr, v, sep, b * g, rep * s, d, l, l, d, d, rep * s * l, l * d, rep * s * d)
    out, exp = to_np(got), to_np(sep)
    assert np.isfinite(exp).all() and np.isfinite(out).all()
    assert_close(out, exp, rtol=1e-4, atol=1e-5)
    # the rows with nothing visible are the plain average of their KV head's V rows
    mean_v = np.repeat(v_np.astype(np.float64).mean(axis=2), rep, axis=1).astype(np.float32)
    for row in (5, s - 1):
        assert_close(out[:, :, row], mean_v, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("kw", [dict(d=32), dict(l=130), dict(last_stride=2)])
def test_attention_declines_what_it_does_not_cover(device, kw):
    import torch
    from rmlk_amd import RmlkError
    kk = _k()
    d, l = kw.get("d", 64), kw.get("l", 128)
    q = torch.zeros(1, 2, 64, d, device=device)
    k = torch.zeros(1, 2, l, d, device=device)
    m = torch.zeros(64, 2 * l, device=device)
    out = torch.zeros_like(q)
    with pytest.raises(RmlkError) as e:
        kk.attention(q, k, k, m, out, 1, 2, 1, 64, l, d, [0, 0, 2 * l, kw.get("last_stride", 1)], 8.0)
    assert e.value.status == -2


@pytest.mark.parametrize("s,l,rep", [(200, 256, 4), (1, 256, 4), (48, 64, 1)])
def test_attention_chain_becomes_one_node(device, s, l, rep):
    """scores -> Div -> Add(mask) -> Softmax -> context over a grouped KV cache: one node; with
    enough query rows it runs the one-kernel attention, a decode step runs the three nodes."""
    from oracle import graph as og
    b, g, d = 1, 2, 64
    h = g * rep
    gb = _builder()
    gb.input("q", np.float32, [b, h, 0, d])
    gb.input("k", np.float32, [b, g, l, d])
    gb.input("v", np.float32, [b, g, l, d])
    gb.input("mask", np.float32, [1, 1, 0, l])
    gb.constant("ax", np.array([2], np.int64))
    gb.constant("eshape", np.array([1, g, rep, 1, 1], np.int64))
    gb.constant("rshape", np.array([b, h, -1, d], np.int64))
    gb.constant("scale", np.array(8.0, np.float32))
    for t in ("k", "v"):
        if rep > 1:
            gb.op("Unsqueeze", [t, "ax"], [t + "u"])
            gb.op("Expand", [t + "u", "eshape"], [t + "e"])
            gb.op("Reshape", [t + "e", "rshape"], [t + "x"])
    kx, vx = ("kx", "vx") if rep > 1 else ("k", "v")
    gb.op("Transpose", [kx], ["kt"]).attr("perm", [0, 1, 3, 2])
    gb.op("MatMul", ["q", "kt"], ["scores"])
    gb.op("Div", ["scores", "scale"], ["scaled"])
    gb.op("Add", ["scaled", "mask"], ["masked"])
    gb.op("Softmax", ["masked"], ["probs"]).attr("axis", -1)
    gb.op("MatMul", ["probs", vx], ["ctx_heads"])
    gb.op("Transpose", ["ctx_heads"], ["ctx"]).attr("perm", [0, 2, 1, 3])   # absorbed as well
    gb.output("ctx")
    graph = gb.build()
    rng = np.random.default_rng(s + l)
    mask = np.triu(np.full((s, l), -np.inf, dtype=np.float32), l - s + 1).reshape(1, 1, s, l)
    feeds = {"q": rng.standard_normal((b, h, s, d), dtype=np.float32),
             "k": rng.standard_normal((b, g, l, d), dtype=np.float32),
             "v": rng.standard_normal((b, g, l, d), dtype=np.float32), "mask": mask}
    a_, b_, n, _ = _run_both(graph, feeds)
    # the scores product (K transpose, KV repeat), the softmax chain, the context product when it
    # carries the KV repeat (plain MatMul otherwise), and the three merged
    assert n == (4 if rep > 1 else 3)
    exp = og.run_graph(graph, feeds)
    assert_close(a_["ctx"], b_["ctx"], rtol=1e-4, atol=1e-5)
    assert_close(a_["ctx"], exp["ctx"], rtol=1e-4, atol=1e-5)


def test_decoder_layer_gives_the_same_bits_every_time(device):
    """Every kernel sums in a fixed order and awaits its own loads: repeated runs of one session on
    the same inputs are bit-identical (the recorded-graph replay depends on it)."""
    from rmlk_amd import graphs, runtime
    graph, feeds = graphs.decoder_layer_graph(seed=5, seq=512)
    inst = runtime.Builder.from_graph(graph).build()
    first = inst.run(feeds)
    for _ in range(12):
        again = inst.run(feeds)
        for name in first:
            assert_exact(again[name], first[name])
    inst.close()


def test_long_prompt_replays_give_the_bits_of_the_eager_run(device):
    """A 2048-token prompt (the causal mask no longer fits the caches, so its loads are slow) through
    a recorded graph: every replay equals the eager run bit for bit. The attention kernel once took
    its prefetched mask from registers that the data had not reached yet, in about one replay of
    twenty at this size."""
    from rmlk_amd import graphs, runtime
    cfg = graphs.LlamaConfig()
    cfg.layers, cfg.vocab = 4, 8192
    prompt_len, max_len = 2048, 2064
    graph = graphs.llama_graph(cfg, seed=4, style="scatter", max_len=max_len)
    inst = runtime.Builder.from_graph(graph).build()
    rng = np.random.default_rng(4)
    inst.set_input("input_ids", rng.integers(0, cfg.vocab, size=(1, prompt_len)).astype(np.int64))
    inst.set_input("position_ids", np.arange(prompt_len, dtype=np.int64).reshape(1, -1))
    for l in range(cfg.layers):
        for kv in ("key", "value"):
            inst.set_input(f"cache.{l}.{kv}", np.zeros((1, cfg.kv_heads, max_len, cfg.head_dim), np.float32))
    names = [f"cache_out.{cfg.layers - 1}.key", "logits"]
    inst.execute()
    first = {n: inst.output(n).copy() for n in names}
    inst.capture()
    for _ in range(10):
        inst.replay()
        inst.sync()
        for n in names:
            assert_exact(inst.output(n), first[n])
    inst.close()


@pytest.mark.parametrize("m,n,k", [(512, 2048, 2048), (512, 2048, 8192), (300, 96, 200), (64, 256, 64)])
def test_matmul_partials_feed_the_norm(device, m, n, k):
    """rmlk_hip_matmul_partials + rmlk_hip_splitk_add_rmsnorm against rmlk_hip_matmul +
    rmlk_hip_add_rmsnorm: the same slabs added in the same order, so the same bits."""
    import ctypes
    import torch
    from rmlk_amd._lib import check, lib
    kk = _k()
    rng = np.random.default_rng(m + n + k)
    a = to_dev(rng.standard_normal((m, k), dtype=np.float32), device)
    w = to_dev(rng.standard_normal((k, n), dtype=np.float32) * np.float32(0.02), device)
    res = to_dev(rng.standard_normal((m, n), dtype=np.float32), device)
    gamma = to_dev(rng.uniform(0.5, 1.5, size=(n,)).astype(np.float32), device)
    stream = torch.cuda.current_stream().cuda_stream
    need = int(lib().rmlk_hip_matmul_partials_workspace_size(kk.FLOAT, m, n, k))
    assert need >= m * n * 4
    ws = torch.empty(need, dtype=torch.uint8, device=device)
    splits = ctypes.c_int32(0)
    check(lib().rmlk_hip_matmul_partials(stream, kk.FLOAT, m, n, k, a.data_ptr(), k, kk.FLOAT, w.data_ptr(), n, 0,
                                         ws.data_ptr(), need, ctypes.byref(splits)),
          "rmlk_hip_matmul_partials")
    assert 1 <= splits.value and splits.value * m * n * 4 <= need
    if k % 4 == 0:
        # K-contiguous weights: the same slabs
        wt = w.t().contiguous()
        ws_t = torch.empty(need, dtype=torch.uint8, device=device)
        splits_t = ctypes.c_int32(0)
        check(lib().rmlk_hip_matmul_partials(stream, kk.FLOAT, m, n, k, a.data_ptr(), k, kk.FLOAT, wt.data_ptr(), k, 1,
                                             ws_t.data_ptr(), need, ctypes.byref(splits_t)),
              "rmlk_hip_matmul_partials")
        assert splits_t.value == splits.value
        used = splits.value * m * n * 4
        assert_exact(to_np(ws_t[:used]), to_np(ws[:used]))
    got_sum, got = torch.empty_like(res), torch.empty_like(res)
    check(lib().rmlk_hip_splitk_add_rmsnorm(stream, kk.FLOAT, m, n, ws.data_ptr(), splits.value, m * n,
                                            res.data_ptr(), gamma.data_ptr(), 1e-5, 0,
                                            got_sum.data_ptr(), got.data_ptr()),
          "rmlk_hip_splitk_add_rmsnorm")
    prod = torch.empty(m, n, device=device)
    kk.matmul(a, w, prod, 1, m, n, k, k, n, n, 0, 0, 0)
    exp_sum, exp = torch.empty_like(res), torch.empty_like(res)
    kk.add_rmsnorm(prod, res, gamma, exp_sum, exp, m, n, 1e-5)
    assert_exact(to_np(got_sum), to_np(exp_sum))
    assert_exact(to_np(got), to_np(exp))


@pytest.mark.parametrize("n,k", [(2048, 2048), (2048, 8192), (3072, 2048), (128256, 2048), (5, 8), (70, 132)])
def test_one_row_product_over_k_contiguous_weights(device, n, k):
    import torch
    kk = _k()
    rng = np.random.default_rng(n + k)
    x_np = rng.standard_normal((k,), dtype=np.float32)
    w_np = rng.standard_normal((k, n), dtype=np.float32) * np.float32(0.02)
    x, w = to_dev(x_np, device), to_dev(w_np, device)
    wt = to_dev(np.ascontiguousarray(w_np.T), device)
    got = torch.full((n,), float("nan"), device=device)
    kk.gemv_kmajor(x, wt, got, n, k)
    sep = torch.empty(n, device=device)
    kk.matmul(x, w, sep, 1, 1, n, k, k, n, n, 0, 0, 0)
    assert_close(to_np(got), to_np(sep), rtol=1e-4, atol=1e-5)
    exp = x_np.astype(np.float64) @ w_np.astype(np.float64)
    assert_close(to_np(got), exp.astype(np.float32), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("n,k,recip", [(3072, 2048, False), (128256, 2048, True), (70, 132, False),
                                       (512, 8192, True), (40, 8, False), (64, 1024, False)])
def test_one_row_products_over_a_row_normalised_on_the_fly(device, n, k, recip):
    """The K-major one-row products over RMSNorm(x) * gamma without storing the normalised row, and
    with a residual added to the result: bit for bit what the norm kernel, the product kernel and
    an Add give one after the other."""
    import torch
    kk = _k()
    rng = np.random.default_rng(n + k)
    x = to_dev(rng.standard_normal((k,), dtype=np.float32) * np.float32(3.0), device)
    gamma = to_dev(rng.uniform(0.5, 1.5, size=(k,)).astype(np.float32), device)
    wt = to_dev(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.05), device)
    res = to_dev(rng.standard_normal((n,), dtype=np.float32), device)
    normed, exp, got = torch.empty(k, device=device), torch.empty(n, device=device), torch.empty(n, device=device)
    kk.rmsnorm(x, gamma, normed, 1, k, 1e-5, recip)
    kk.gemv_kmajor(normed, wt, exp, n, k)
    kk.gemv_kmajor_normed(x, gamma, wt, got, n, k, 1e-5, recip)
    assert_exact(to_np(got), to_np(exp))
    # residual epilogue
    plain, summed = torch.empty(n, device=device), torch.empty(n, device=device)
    kk.gemv_kmajor(x, wt, plain, n, k)
    kk.binary(kk.ADD, plain, res, summed, [n], [1], [1])
    kk.gemv_kmajor_add(x, wt, res, got, n, k)
    assert_exact(to_np(got), to_np(summed))
    if n % 2 == 0:
        half = n // 2
        kk.gemv_kmajor_swiglu(normed, wt, exp[:half], half, k, 0, half)
        kk.gemv_kmajor_swiglu_normed(x, gamma, wt, got[:half], half, k, 0, half, 1e-5, recip)
        assert_exact(to_np(got[:half]), to_np(exp[:half]))


def test_one_row_products_over_a_normalised_row_decline_what_they_do_not_cover(device):
    import torch
    from rmlk_amd import RmlkError
    kk = _k()
    n, k = 8, 16
    x = torch.ones(k + 4, device=device)
    wt = torch.ones(n * k, device=device)
    gamma = torch.ones(k + 4, device=device)
    y = torch.empty(n, device=device)
    kk.gemv_kmajor_normed(x, gamma, wt, y, 0, k, 1e-5)                      # nothing to do
    with pytest.raises(RmlkError):                                          # row longer than a block normalises
        big = torch.ones(16384, device=device)
        kk.gemv_kmajor_normed(big, big, torch.ones(4 * 16384, device=device), y[:4], 4, 16384, 1e-5)
    with pytest.raises(RmlkError):                                          # K no multiple of 4
        kk.gemv_kmajor_normed(x, gamma, wt, y, n, 14, 1e-5)
    with pytest.raises(RmlkError):                                          # x not 16-byte aligned
        kk.gemv_kmajor_normed(x[1:], gamma, wt, y, n, k, 1e-5)
    with pytest.raises(RmlkError):                                          # gamma not 16-byte aligned
        kk.gemv_kmajor_normed(x, gamma[1:], wt, y, n, k, 1e-5)
    with pytest.raises(RmlkError):
        kk.gemv_kmajor_swiglu_normed(x, gamma[1:], wt, y, n // 2, k, 0, n // 2, 1e-5)
    with pytest.raises(RmlkError):                                          # x not 16-byte aligned
        kk.gemv_kmajor_add(x[1:], wt, y, y, n, k)


@pytest.mark.parametrize("n,k,gate_first", [(8192, 2048, True), (512, 256, False), (7, 64, True)])
def test_one_row_gate_up_swiglu_over_k_contiguous_weights(device, n, k, gate_first):
    import torch
    kk = _k()
    rng = np.random.default_rng(n + k)
    x_np = rng.standard_normal((k,), dtype=np.float32)
    wt_np = rng.standard_normal((2 * n, k), dtype=np.float32) * np.float32(0.05)
    x, wt = to_dev(x_np, device), to_dev(wt_np, device)
    go, uo = (0, n) if gate_first else (n, 0)
    got = torch.full((n,), float("nan"), device=device)
    kk.gemv_kmajor_swiglu(x, wt, got, n, k, go, uo)
    both = torch.empty(2 * n, device=device)
    kk.gemv_kmajor(x, wt, both, 2 * n, k)
    sep = torch.empty(n, device=device)
    kk.swiglu(both[go:go + n].contiguous(), both[uo:uo + n].contiguous(), sep)
    assert_close(to_np(got), to_np(sep), rtol=1e-4, atol=1e-5)
    g64 = wt_np[go:go + n].astype(np.float64) @ x_np.astype(np.float64)
    u64 = wt_np[uo:uo + n].astype(np.float64) @ x_np.astype(np.float64)
    assert_close(to_np(got), (g64 / (1.0 + np.exp(-g64)) * u64).astype(np.float32), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("b,g,rep,s,l,mask_shape,mul", [
    (1, 8, 4, 1, 640, (1, 1, 1, 640), False),      # a decode step of the 1B shape
    (2, 2, 3, 2, 130, (2, 1, 2, 130), True),       # ragged last chunk, per-batch mask, two query rows
    (1, 1, 1, 1, 5, (1, 1, 1, 5), False),
    (1, 2, 16, 1, 200, (1, 32, 1, 200), True),     # 16 query heads per KV head, per-head mask
])
def test_attention_few_rows_matches_separate_kernels(device, b, g, rep, s, l, mask_shape, mul):
    import torch
    kk = _k()
    h, d = g * rep, 64
    rng = np.random.default_rng(b * 100 + s + l)
    q_np = rng.standard_normal((b, h, s, d), dtype=np.float32)
    k_np = rng.standard_normal((b, g, l, d), dtype=np.float32)
    v_np = rng.standard_normal((b, g, l, d), dtype=np.float32)
    m_np = rng.standard_normal(mask_shape, dtype=np.float32)
    m_np[..., l - l // 3:] = -np.inf          # the unwritten tail of a cache
    scale = 8.0 if not mul else 0.125
    q, k, v, m = (to_dev(x, device) for x in (q_np, k_np, v_np, m_np))
    full = [b, h, s, l]
    ms = bcast_strides(list(mask_shape), full)
    got = torch.full((b, h, s, d), float("nan"), device=device)
    kk.attention_few_rows(q, k, v, m, got, b, g, rep, s, l, d, ms, scale, mul)
    assert_close(to_np(got), _attention_reference(q_np, k_np, v_np, m_np, scale, mul), rtol=1e-4, atol=1e-5)
    moved = torch.full((b, s, h, d), float("nan"), device=device)
    kk.attention_few_rows(q, k, v, m, moved, b, g, rep, s, l, d, ms, scale, mul, out_seq_major=True)
    assert_exact(to_np(moved), to_np(got).transpose(0, 2, 1, 3))


@pytest.mark.parametrize("b,g,rep,s,l,mask_shape", [
    (1, 8, 4, 1, 640, (1, 1, 1, 640)),       # a decode step of the 1B shape
    (1, 8, 4, 1, 2048, (1, 1, 1, 2048)),     # 32 chunks
    (2, 2, 3, 2, 130, (2, 1, 2, 130)),       # ragged last chunk, per-batch mask, two query rows
    (1, 1, 1, 1, 5, (1, 1, 1, 5)),           # one chunk: every block is the last
    (1, 2, 16, 1, 200, (1, 32, 1, 200)),     # 16 query heads per KV head
    (3, 8, 2, 1, 4500, (3, 1, 1, 4500)),     # more chunks than a wavefront has lanes
])
def test_attention_few_rows_in_one_launch_is_bit_identical(device, b, g, rep, s, l, mask_shape):
    """The last block of a KV head merges its chunks: same numbers as the two-kernel call, and the
    counters are zero again, call after call with the same counters."""
    import torch
    kk = _k()
    h, d = g * rep, 64
    rng = np.random.default_rng(b * 100 + s + l)
    q, k, v = (to_dev(rng.standard_normal(sh, dtype=np.float32), device)
               for sh in ((b, h, s, d), (b, g, l, d), (b, g, l, d)))
    m_np = rng.standard_normal(mask_shape, dtype=np.float32)
    m_np[..., l - l // 3:] = -np.inf
    m = to_dev(m_np, device)
    ms = bcast_strides(list(mask_shape), [b, h, s, l])
    exp = torch.full((b, h, s, d), float("nan"), device=device)
    kk.attention_few_rows(q, k, v, m, exp, b, g, rep, s, l, d, ms, 8.0)
    counters = torch.zeros(b * g + 3, dtype=torch.int32, device=device)
    counters[b * g:] = 77     # not the kernel's
    for seq_major in (False, True, False):
        got = torch.full((b, s, h, d) if seq_major else (b, h, s, d), float("nan"), device=device)
        kk.attention_few_rows_one_launch(q, k, v, m, got, counters, b, g, rep, s, l, d, ms, 8.0,
                                         out_seq_major=seq_major)
        want = to_np(exp).transpose(0, 2, 1, 3) if seq_major else to_np(exp)
        assert_exact(to_np(got), want)
        assert to_np(counters).tolist() == [0] * (b * g) + [77] * 3


def test_attention_few_rows_declines_many_rows(device):
    import torch
    from rmlk_amd import RmlkError
    kk = _k()
    q = torch.zeros(1, 8, 5, 64, device=device)
    k = torch.zeros(1, 2, 64, 64, device=device)
    m = torch.zeros(5, 64, device=device)
    with pytest.raises(RmlkError):
        kk.attention_few_rows(q, k, k, m, torch.zeros_like(q), 1, 2, 4, 5, 64, 64, [0, 0, 64, 1], 8.0)

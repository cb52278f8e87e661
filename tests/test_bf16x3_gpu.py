"""Many-row products over bfloat16 weights on the bf16 matrix cores (rmlk_hip_bf16x3_split,
rmlk_hip_matmul_bf16x3, rmlk_hip_matmul_bf16x3_swiglu; sessions built with bf16_pieces=True).

The reference multiplies in fp32 (cuBLAS, cuda/src/kernels/gemm.rs:191-232). Here the fp32 operand is
split into three bfloat16 pieces whose sum it is EXACTLY, every piece-times-weight product is exact in
fp32, and only the fp32 accumulation rounds. What pins that:
  - the pieces add up to the operand bit for bit (any float, subnormal results aside), Inf / NaN stay;
  - products whose every partial sum is an integer below 2^24 are exact whatever the order: bit-equal
    to the float64 product - a dropped piece, a wrong row, unit or K range fails this;
  - on full-mantissa data the error against float64 is that of fp32 accumulation (a dropped `lo`
    piece alone would cost 2^-16 relative);
  - the SwiGLU form equals rmlk_hip_swiglu over the two plain products bit for bit.
"""
import numpy as np
import pytest

from helpers import assert_close, assert_exact, to_dev, to_np

pytestmark = pytest.mark.gpu


def _k():
    from rmlk_amd import kernels
    return kernels


def _bf16_weights(w_np, device):
    import torch
    return to_dev(w_np.astype(np.float32), device).to(torch.bfloat16)


def _planes(pieces, m, k):
    """[3][m_pad][k] float64 values of the pieces tensor."""
    import torch
    m_pad = (m + 127) // 128 * 128
    return pieces.view(torch.bfloat16).reshape(3, m_pad, k).to(torch.float64).cpu().numpy()


def test_pieces_add_up_to_the_operand_exactly(device):
    import torch
    kk = _k()
    rng = np.random.default_rng(0)
    m, k = 130, 64
    a = (rng.standard_normal((m, k)) * np.exp(rng.uniform(-30, 30, size=(m, k)))).astype(np.float32)
    a[0, :8] = [0.0, -0.0, 1.0, -1.0, np.float32(1) + np.float32(2.0 ** -23), 3.0e38, -3.0e38, 2.0 ** -100]
    a[1, :3] = [np.inf, -np.inf, np.nan]
    pieces = kk.bf16x3_split(to_dev(a, device))
    torch.cuda.synchronize()
    p = _planes(pieces, m, k)
    assert p.shape == (3, 256, k)
    assert not p[:, m:, :].any()                                  # padding rows
    finite = np.isfinite(a)
    total = p[0, :m] + p[1, :m] + p[2, :m]                       # (float64: exact)
    assert np.array_equal(total[finite], a.astype(np.float64)[finite])
    # every piece has eight significant bits at most and they do not overlap
    assert np.all(np.abs(p[1, :m][finite]) <= np.abs(p[0, :m][finite]) * 2.0 ** -7)
    assert np.all(np.abs(p[2, :m][finite]) <= np.abs(p[0, :m][finite]) * 2.0 ** -15)
    assert np.isposinf(p[0, 1, 0]) and np.isneginf(p[0, 1, 1]) and np.isnan(p[0, 1, 2])
    assert not p[1:, 1, :3].any()


@pytest.mark.parametrize("m,n,k,splits", [
    (64, 128, 32, 1),          # one tile, one K step
    (128, 256, 64, 2),         # the 256-column tile is not picked (too few tiles): 128-column tiles, a slab per K step
    (130, 384, 96, 1),         # rows past the end of the last tile, three K steps (fewer than the stages)
    (200, 256, 512, 2),
    (512, 2048, 2048, 4),      # the output projection of a 512-token prefill
    (512, 3072, 2048, 2),      # q | k | v
    (256, 32768, 256, 1),      # 256-column tiles, one block per compute unit (three stages)
    (384, 65536, 64, 1),       # 256-column tiles, more blocks than compute units (two stages)
])
def test_products_of_small_integers_are_exact(device, m, n, k, splits):
    import torch
    kk = _k()
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(-8, 9, size=(m, k)).astype(np.float32)
    w = rng.integers(-4, 5, size=(n, k)).astype(np.float32)
    a_d, w_d = to_dev(a, device), _bf16_weights(w, device)
    pieces = kk.bf16x3_split(a_d)
    out = torch.full((splits, m, n), np.nan, dtype=torch.float32, device=device)
    kk.matmul_bf16x3(pieces, w_d, out, m, n, k, splits)
    got = to_np(out)
    per = k // splits
    for s in range(splits):
        exp = a[:, s * per:(s + 1) * per].astype(np.float64) @ w[:, s * per:(s + 1) * per].astype(np.float64).T
        assert np.array_equal(got[s].astype(np.float64), exp), f"slab {s}"


def test_random_sizes_of_small_integers_are_exact(device):
    """Forty random sizes (any m, n in whole 128-column tiles, K in whole steps, any slab count that
    cuts K into whole steps), plain and SwiGLU form: every tile shape, stage count, step count below
    and above the number of stages, padded rows."""
    import torch
    kk = _k()
    rng = np.random.default_rng(77)
    for case in range(40):
        m = int(rng.integers(1, 700))
        n = 128 * int(rng.integers(1, 40)) if case % 4 else 256 * int(rng.integers(100, 300))
        steps = int(rng.integers(1, 60))
        splits = int(rng.choice([s for s in (1, 2, 3, 4, 8) if steps % s == 0]))
        k = 32 * steps
        if m * n > 40e6:
            m = max(1, int(40e6 // n))
        a = rng.integers(-8, 9, size=(m, k)).astype(np.float32)
        w = rng.integers(-4, 5, size=(n, k)).astype(np.float32)
        a_d, w_d = to_dev(a, device), _bf16_weights(w, device)
        pieces = kk.bf16x3_split(a_d)
        out = torch.full((splits, m, n), np.nan, dtype=torch.float32, device=device)
        kk.matmul_bf16x3(pieces, w_d, out, m, n, k, splits)
        got = out.to(torch.float64).sum(0)
        exp = a_d.to(torch.float64) @ w_d.to(torch.float64).T
        assert torch.equal(got, exp), (case, m, n, k, splits)
        if n % 256 == 0:
            half = n // 2
            act = torch.full((m, half), np.nan, dtype=torch.float32, device=device)
            kk.matmul_bf16x3_swiglu(pieces, w_d, act, m, half, k, half, 0)
            gate, up = exp[:, half:], exp[:, :half]
            ref = (gate / (1 + torch.exp(-gate)) * up).to(torch.float32)
            assert torch.allclose(act, ref, rtol=1e-5, atol=1e-5), (case, m, n, k, "swiglu")


@pytest.mark.parametrize("m,n,k", [(512, 2048, 2048), (100, 640, 8192), (512, 16384, 256)])
def test_full_mantissa_products_have_the_error_of_fp32_accumulation(device, m, n, k):
    import torch
    kk = _k()
    rng = np.random.default_rng(k)
    a = (rng.standard_normal((m, k)) * 1.7).astype(np.float32)
    w_d = _bf16_weights(rng.standard_normal((n, k)) * 0.05, device)
    a_d = to_dev(a, device)
    splits = kk.bf16x3_splits(m, n, k)
    assert splits >= 1
    out = torch.zeros((splits, m, n), dtype=torch.float32, device=device)
    kk.matmul_bf16x3(kk.bf16x3_split(a_d), w_d, out, m, n, k, splits)
    got = out.to(torch.float64).sum(0)
    exp = a_d.to(torch.float64) @ w_d.to(torch.float64).T
    scale = a_d.to(torch.float64).abs() @ w_d.to(torch.float64).abs().T
    err = ((got - exp).abs() / scale).max().item()
    # fp32 accumulation of K terms in blocks: a few 2^-24 of sum |a||w| (a dropped `lo` piece alone: 2^-16)
    assert err < 1e-6, err


@pytest.mark.parametrize("m,n,k,gate_first", [
    (512, 8192, 2048, True),     # gate / up of a 512-token prefill: 256-row tiles of W, 128 columns out
    (512, 8192, 2048, False),
    (128, 192, 64, True),        # n % 128 != 0: the 128-row tile, 64 columns out
    (70, 256, 96, False),
])
def test_swiglu_form_equals_the_two_products_and_the_activation(device, m, n, k, gate_first):
    import torch
    kk = _k()
    rng = np.random.default_rng(n + k)
    a_d = to_dev(rng.standard_normal((m, k)).astype(np.float32), device)
    w_d = _bf16_weights(rng.standard_normal((2 * n + 128, k)) * 0.06, device)   # (rows behind both blocks)
    gate_row, up_row = (0, n) if gate_first else (n, 0)
    pieces = kk.bf16x3_split(a_d)
    got = torch.zeros((m, n), dtype=torch.float32, device=device)
    kk.matmul_bf16x3_swiglu(pieces, w_d, got, m, n, k, gate_row, up_row)
    # the same launch storing the pieces of its result: the same floats, and the pieces of those
    m_pad = (m + 127) // 128 * 128
    again = torch.zeros((m, n), dtype=torch.float32, device=device)
    act = torch.zeros(3 * m_pad * n, dtype=torch.int16, device=device)
    kk.matmul_bf16x3_swiglu(pieces, w_d, again, m, n, k, gate_row, up_row, out_pieces=act)
    assert_exact(to_np(again), to_np(got))
    assert torch.equal(act.reshape(3, m_pad, n)[:, :m], kk.bf16x3_split(got).reshape(3, m_pad, n)[:, :m])
    exp64 = None
    if n % 128 == 0:
        # the same accumulation order in the plain product: bit for bit
        gate = torch.zeros((m, n), dtype=torch.float32, device=device)
        up = torch.zeros((m, n), dtype=torch.float32, device=device)
        kk.matmul_bf16x3(pieces, w_d[gate_row:gate_row + n], gate, m, n, k)
        kk.matmul_bf16x3(pieces, w_d[up_row:up_row + n], up, m, n, k)
        exp = torch.zeros((m, n), dtype=torch.float32, device=device)
        kk.swiglu(gate, up, exp)
        assert_exact(to_np(got), to_np(exp))
    g64 = a_d.to(torch.float64) @ w_d[gate_row:gate_row + n].to(torch.float64).T
    u64 = a_d.to(torch.float64) @ w_d[up_row:up_row + n].to(torch.float64).T
    exp64 = (g64 / (1 + torch.exp(-g64)) * u64).cpu().numpy()
    # (gate and up are sums of k terms of size ~0.06 each, |gate|, |up| up to ~10: fp32 accumulation
    # leaves ~1e-6 of that on values that may themselves be near zero)
    assert_close(to_np(got), exp64.astype(np.float32), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("m,k,widths", [(300, 256, (2048, 512, 512)), (64, 64, (96, 32)), (2048, 128, (256,)),
                                        (130, 96, (32, 32, 32, 160))])
def test_grouped_product_sends_column_blocks_to_their_members(device, m, k, widths):
    """One launch over the joint matrix [sum(widths), k]; every member's output equals the plain
    product over its rows of the matrix bit for bit (same K order), small integers exactly."""
    import torch
    from rmlk_amd._lib import RmlkError
    kk = _k()
    rng = np.random.default_rng(sum(widths) + m)
    n = sum(widths)
    a = rng.integers(-8, 9, size=(m, k)).astype(np.float32)
    w = rng.integers(-4, 5, size=(n, k)).astype(np.float32)
    a_d, w_d = to_dev(a, device), _bf16_weights(w, device)
    pieces = kk.bf16x3_split(a_d)
    outs = [torch.full((m, wd), np.nan, dtype=torch.float32, device=device) for wd in widths]
    kk.matmul_bf16x3_grouped(pieces, w_d, outs, m, k, list(widths))
    first = 0
    for wd, out in zip(widths, outs):
        exp = a.astype(np.float64) @ w[first:first + wd].astype(np.float64).T
        assert np.array_equal(to_np(out).astype(np.float64), exp), (first, wd)
        first += wd
    # full-mantissa operands: the joint launch against the plain product over the joint matrix
    a_d = to_dev(rng.standard_normal((m, k)).astype(np.float32), device)
    w_d = _bf16_weights(rng.standard_normal((n, k)) * 0.05, device)
    pieces = kk.bf16x3_split(a_d)
    kk.matmul_bf16x3_grouped(pieces, w_d, outs, m, k, list(widths))
    whole = torch.zeros((m, n), dtype=torch.float32, device=device)
    kk.matmul_bf16x3(pieces, w_d, whole, m, n, k)
    first = 0
    for wd, out in zip(widths, outs):
        assert_exact(to_np(out), to_np(whole[:, first:first + wd].contiguous()))
        first += wd
    with pytest.raises(RmlkError) as e:       # a boundary inside a 32-column block
        kk.matmul_bf16x3_grouped(pieces, w_d, outs[:1] * 2, m, k, [48, n - 48])
    assert e.value.status == -2


@pytest.mark.parametrize("rows,cols,splits,with_add", [(512, 2048, 4, True), (70, 256, 1, False), (130, 8192, 2, True),
                                                        (2048, 512, 1, True)])
def test_norm_that_stores_its_result_as_pieces(device, rows, cols, splits, with_add):
    """rmlk_hip_rmsnorm_pieces: `out` and `sum_out` are the bits of the norm entry points, and the
    pieces are those that rmlk_hip_bf16x3_split makes of `out` (padding rows aside)."""
    import torch
    kk = _k()
    rng = np.random.default_rng(rows + cols)
    x = to_dev(rng.standard_normal((splits, rows, cols)).astype(np.float32), device)
    add = to_dev(rng.standard_normal((rows, cols)).astype(np.float32), device) if with_add else None
    gamma = to_dev((1 + 0.1 * rng.standard_normal(cols)).astype(np.float32), device)
    out, exp = torch.zeros((rows, cols), device=device), torch.zeros((rows, cols), device=device)
    total, exp_total = torch.zeros((rows, cols), device=device), torch.zeros((rows, cols), device=device)
    m_pad = (rows + 127) // 128 * 128
    pieces = torch.zeros(3 * m_pad * cols, dtype=torch.int16, device=device)
    kk.rmsnorm_pieces(x, gamma, 1e-5, out, pieces, add=add, sum_out=total if with_add else None, splits=splits)
    if with_add:
        from rmlk_amd._lib import check, lib
        check(lib().rmlk_hip_splitk_add_rmsnorm(torch.cuda.current_stream().cuda_stream, kk.FLOAT, rows, cols,
                                                x.data_ptr(), splits, rows * cols, add.data_ptr(), gamma.data_ptr(),
                                                1e-5, 0, exp_total.data_ptr(), exp.data_ptr()),
              "rmlk_hip_splitk_add_rmsnorm")
        assert_exact(to_np(total), to_np(exp_total))
    else:
        kk.rmsnorm(x[0], gamma, exp, rows, cols, 1e-5)
    assert_exact(to_np(out), to_np(exp))
    want = kk.bf16x3_split(exp).reshape(3, m_pad, cols)[:, :rows]
    assert torch.equal(pieces.reshape(3, m_pad, cols)[:, :rows], want)


@pytest.mark.parametrize("b,g,rep,s,l", [(1, 8, 4, 512, 640),      # the 512-token prefill into a 640-long cache
                                         (2, 2, 2, 192, 256),      # two sequences, tiles of the last rows half empty
                                         (1, 8, 4, 2048, 2048)])   # more blocks than compute units, chunks skipped
def test_attention_that_stores_its_result_as_pieces(device, b, g, rep, s, l):
    """rmlk_hip_attention_ws_pieces: the [B, S, H, D] result bit for bit as without the pieces, and the
    pieces those that rmlk_hip_bf16x3_split makes of the [B * S, H * D] matrix it is."""
    import torch
    kk = _k()
    h, d = g * rep, 64
    rng = np.random.default_rng(s + l)
    q, k, v = (to_dev(rng.standard_normal(sh, dtype=np.float32), device)
               for sh in ((b, h, s, d), (b, g, l, d), (b, g, l, d)))
    mask = np.where(np.arange(l)[None, :] <= np.arange(s)[:, None] + (l - s) // 2, 0.0, -np.inf).astype(np.float32)
    m = to_dev(mask.reshape(1, 1, s, l), device)
    ms = [0, 0, l, 1]
    plain = torch.full((b, s, h, d), 7.0, device=device)
    kk.attention_skipping(q, k, v, m, plain, b, g, rep, s, l, d, ms, 8.0, False, out_seq_major=True)
    rows, cols = b * s, h * d
    m_pad = (rows + 127) // 128 * 128
    got = torch.full((b, s, h, d), 9.0, device=device)
    pieces = torch.zeros(3 * m_pad * cols, dtype=torch.int16, device=device)
    kk.attention_skipping(q, k, v, m, got, b, g, rep, s, l, d, ms, 8.0, False, out_seq_major=True, out_pieces=pieces)
    assert_exact(to_np(got), to_np(plain))
    want = kk.bf16x3_split(plain.reshape(rows, cols)).reshape(3, m_pad, cols)[:, :rows]
    assert torch.equal(pieces.reshape(3, m_pad, cols)[:, :rows], want)
    # the same over a map of the mask made beforehand (rmlk_hip_attention_mapped_pieces), twice
    tile_map = kk.attention_map(m, b, g, rep, s, l, d, ms)
    assert tile_map is not None
    for _ in range(2):
        again = torch.full((b, s, h, d), 9.0, device=device)
        pieces2 = torch.zeros(3 * m_pad * cols, dtype=torch.int16, device=device)
        kk.attention_mapped(q, k, v, m, again, tile_map, b, g, rep, s, l, d, ms, 8.0, False, out_seq_major=True,
                            out_pieces=pieces2)
        assert_exact(to_np(again), to_np(plain))
        assert torch.equal(pieces2.reshape(3, m_pad, cols)[:, :rows], want)


def test_infinities_and_nans_arrive_as_from_an_fp32_product(device):
    import torch
    kk = _k()
    rng = np.random.default_rng(5)
    m, n, k = 64, 128, 64
    a = rng.standard_normal((m, k)).astype(np.float32)
    a[3, 5], a[7, 0], a[9, 63] = np.inf, np.nan, -np.inf
    w = rng.standard_normal((n, k)).astype(np.float32)
    w[:, 63] = np.abs(w[:, 63]) + 0.5      # -inf * positive: -inf everywhere in row 9
    w[10, 5] = 0.0                          # inf * 0: NaN
    a_d, w_d = to_dev(a, device), _bf16_weights(w, device)
    out = torch.zeros((m, n), dtype=torch.float32, device=device)
    kk.matmul_bf16x3(kk.bf16x3_split(a_d), w_d, out, m, n, k)
    got = to_np(out)
    exp = to_np(a_d @ w_d.to(torch.float32).T)
    assert np.array_equal(np.isnan(got), np.isnan(exp))
    assert np.array_equal(np.isposinf(got), np.isposinf(exp))
    assert np.array_equal(np.isneginf(got), np.isneginf(exp))
    assert np.isnan(got[7]).all() and np.isneginf(got[9]).all() and np.isnan(got[3, 10])


def test_sizes_the_kernels_do_not_take_are_refused(device):
    import torch
    from rmlk_amd._lib import RmlkError
    kk = _k()
    a = torch.zeros((64, 64), device=device)
    w = torch.zeros((256, 64), dtype=torch.bfloat16, device=device)
    pieces = kk.bf16x3_split(a)
    out = torch.zeros((4, 64, 256), device=device)
    assert kk.bf16x3_splits(64, 100, 64) == 0 and kk.bf16x3_splits(64, 128, 40) == 0
    for args in ((64, 100, 64, 1),       # n not in whole tiles
                 (64, 128, 40, 1),       # K steps not whole
                 (64, 128, 64, 4)):      # slabs of half a K step
        with pytest.raises(RmlkError) as e:
            kk.matmul_bf16x3(pieces, w, out, *args)
        assert e.value.status == -2
    with pytest.raises(RmlkError) as e:
        kk.matmul_bf16x3_swiglu(pieces, w, out, 64, 96, 64, 0, 96)
    assert e.value.status == -2
    with pytest.raises(RmlkError) as e:
        kk.matmul_bf16x3(pieces, w, out, 64, 128, 64, 0)
    assert e.value.status == -5
    kk.matmul_bf16x3(pieces, w, out, 0, 128, 64, 1)     # nothing to do: fine


@pytest.mark.parametrize("style", ["scatter", "concat"])
def test_llama_prefill_with_pieces_matches_the_fp32_session(device, style):
    """A Llama-shaped graph whose weights are bfloat16 values, 128 tokens of prefill and three decode
    steps: the session with bf16_pieces sends every product of the prefill to the bf16 matrix cores
    (q|k|v, o, gate|up, down per layer and the lm-head), none of the decode steps', and agrees with
    the fp32 session to fp32 rounding; recorded into a graph it replays to the same values."""
    from rmlk_amd import graphs, runtime
    cfg = graphs.LlamaConfig(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=1024)
    max_len = 160
    graph = graphs.llama_graph(cfg, seed=11, style=style, max_len=max_len, bf16_values=True)
    fast = runtime.Builder.from_graph(graph).build(0, bf16_pieces=True)
    plain = runtime.Builder.from_graph(graph).build(0)
    assert fast.weights_16bit == plain.weights_16bit == 4 * cfg.layers + 1
    rng = np.random.default_rng(8)
    ids, past_len, outs = rng.integers(0, cfg.vocab, size=128), 0, {"fast": None, "plain": None}

    def feeds_for(ids, past, past_len):
        if style == "concat":
            return graphs.llama_concat_inputs(cfg, ids, past, past_len)
        f = {"input_ids": ids.reshape(1, -1).astype(np.int64),
             "position_ids": np.arange(past_len, past_len + ids.size, dtype=np.int64).reshape(1, -1)}
        for l in range(cfg.layers):
            for kv in ("key", "value"):
                f[f"cache.{l}.{kv}"] = (past[f"cache_out.{l}.{kv}"] if past is not None else
                                        np.zeros((1, cfg.kv_heads, max_len, cfg.head_dim), np.float32))
        return f

    for step in range(4):
        outs["fast"] = fast.run(feeds_for(ids, outs["fast"], past_len))
        outs["plain"] = plain.run(feeds_for(ids, outs["plain"], past_len))
        assert fast.products_bf16_pieces == (4 * cfg.layers + 1 if step == 0 else 0)
        assert plain.products_bf16_pieces == 0
        got, exp = outs["fast"]["logits"], outs["plain"]["logits"]
        assert_close(got, exp, rtol=1e-4, atol=2e-5)
        tok = int(np.argmax(got[0, -1]))
        assert tok == int(np.argmax(exp[0, -1]))
        past_len += ids.size
        ids = np.array([tok])
    fast.close()
    plain.close()

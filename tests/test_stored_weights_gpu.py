"""Constant weights stored as 16-bit values (IEEE half, bfloat16) under fp32 arithmetic.

The reference holds fp32 only (its f16 kernel symbols exist but its provider cannot run them), so
there are no reference vectors for this; the bar is what the storage promises:
  - rmlk_hip_store_weights rounds like the oracle's store_weights (itself pinned against closed
    forms and torch's CPU conversion), bit for bit;
  - a many-row product over stored weights EQUALS the fp32 product over the widened weights
    (assert_exact): the same kernels run behind the widening;
  - a one-row product forms its sums in another order than the fp32 kernel: it is held to the
    float64 oracle over the widened weights at the per-op tolerance (rtol 1e-4 / atol 1e-5);
  - a session built with 16-bit weight storage gives what the fp32 session gives on a graph whose
    weights were rounded beforehand, and what the oracle gives on that graph.
"""
import ctypes

import numpy as np
import pytest

from helpers import assert_close, assert_exact, to_dev, to_np

pytestmark = pytest.mark.gpu

STORAGES = ["f16", "bf16"]


def _k():
    from rmlk_amd import kernels
    return kernels


def _torch_dtype(storage):
    import torch
    return {"f16": torch.float16, "bf16": torch.bfloat16}[storage]


def _stored(w_np, storage, device):
    """(device tensor of 16-bit weights, the same values widened to float32 as numpy)."""
    import torch
    from oracle import ops
    kk = _k()
    w = to_dev(w_np, device)
    st = kk.store_weights(w, _torch_dtype(storage))
    wide = st.to(torch.float32)
    assert_exact(to_np(wide), ops.store_weights(w_np, storage))
    return st, to_np(wide)


@pytest.mark.parametrize("storage", STORAGES)
def test_store_weights_rounds_like_the_oracle(device, storage):
    import torch
    from oracle import ops
    kk = _k()
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2 ** 32, size=1 << 18, dtype=np.uint64).astype(np.uint32)
    special = np.array([0x3F808000, 0x3F818000, 0x3F808001, 0x3F807FFF, 0x3FFF8000, 0x7F7FFFFF, 0x80000000,
                        0x00000001, 0xFF800000, 0x7F800000, 0x45001000, 0x45003000, 0x477FF000, 0x33000000,
                        0x33400000], dtype=np.uint32)
    x_np = np.concatenate([special, bits]).view(np.float32)
    got = kk.store_weights(to_dev(x_np, device), _torch_dtype(storage)).to(torch.float32)
    exp = ops.store_weights(x_np, storage)
    nan = np.isnan(exp)
    assert np.array_equal(np.isnan(to_np(got)), nan)
    assert_exact(to_np(got)[~nan], exp[~nan])
    weights = (rng.standard_normal(100001) * 0.02).astype(np.float32)
    assert_exact(to_np(kk.store_weights(to_dev(weights, device), _torch_dtype(storage)).to(torch.float32)),
                 ops.store_weights(weights, storage))
    empty = kk.store_weights(torch.empty(0, device=device), _torch_dtype(storage))
    assert empty.numel() == 0


# k = 2048: one chunk of four units per lane; 8192: chunks of eight; 4096 + 8: a whole chunk and a
# partial one; 264, 8: less than a chunk; n = 7: a block whose last wavefront has no column
@pytest.mark.parametrize("n,k", [(3072, 2048), (2048, 8192), (512, 4104), (7, 264), (64, 8), (33, 2056)])
@pytest.mark.parametrize("storage", STORAGES)
def test_one_row_products_over_stored_weights(device, storage, n, k):
    import torch
    kk = _k()
    rng = np.random.default_rng(n * 7 + k)
    x_np = rng.standard_normal((k,), dtype=np.float32)
    res_np = rng.standard_normal((n,), dtype=np.float32)
    gamma_np = rng.uniform(0.5, 1.5, size=(k,)).astype(np.float32)
    wt, wide = _stored(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.05), storage, device)
    x, res, gamma = to_dev(x_np, device), to_dev(res_np, device), to_dev(gamma_np, device)
    wide_dev = to_dev(wide, device)
    exp64 = wide.astype(np.float64) @ x_np.astype(np.float64)

    got = torch.full((n,), float("nan"), device=device)
    kk.gemv_kmajor(x, wt, got, n, k)
    assert_close(to_np(got), exp64.astype(np.float32), rtol=1e-4, atol=1e-5 * np.sqrt(k))
    # the fp32 kernel over the widened weights: the same numbers up to the order of the sum
    f32 = torch.empty(n, device=device)
    kk.gemv_kmajor(x, wide_dev, f32, n, k)
    assert_close(to_np(got), to_np(f32), rtol=1e-4, atol=1e-5 * np.sqrt(k))

    kk.gemv_kmajor_add(x, wt, res, got, n, k)
    assert_close(to_np(got), (exp64 + res_np).astype(np.float32), rtol=1e-4, atol=1e-5 * np.sqrt(k))

    if k <= 8192:
        eps = 1e-5
        x64 = x_np.astype(np.float64)
        normed = (x64 / np.sqrt(np.mean(x64 * x64) + eps) * gamma_np).astype(np.float32)
        kk.gemv_kmajor_normed(x, gamma, wt, got, n, k, eps)
        assert_close(to_np(got), (wide.astype(np.float64) @ normed.astype(np.float64)).astype(np.float32),
                     rtol=1e-4, atol=1e-5 * np.sqrt(k))
        # bit for bit the norm kernel followed by the product over the same stored weights
        row = torch.empty(k, device=device)
        kk.rmsnorm(x, gamma, row, 1, k, eps, False)
        sep = torch.empty(n, device=device)
        kk.gemv_kmajor(row, wt, sep, n, k)
        assert_exact(to_np(got), to_np(sep))


@pytest.mark.parametrize("n,k,gate_first", [(8192, 2048, True), (512, 8192, False), (7, 64, True)])
@pytest.mark.parametrize("storage", STORAGES)
def test_one_row_gate_up_swiglu_over_stored_weights(device, storage, n, k, gate_first):
    import torch
    kk = _k()
    rng = np.random.default_rng(n + k)
    x_np = rng.standard_normal((k,), dtype=np.float32)
    gamma_np = rng.uniform(0.5, 1.5, size=(k,)).astype(np.float32)
    wt, wide = _stored(rng.standard_normal((2 * n, k), dtype=np.float32) * np.float32(0.05), storage, device)
    x, gamma = to_dev(x_np, device), to_dev(gamma_np, device)
    go, uo = (0, n) if gate_first else (n, 0)

    def swiglu64(row):
        g64 = wide[go:go + n].astype(np.float64) @ row.astype(np.float64)
        u64 = wide[uo:uo + n].astype(np.float64) @ row.astype(np.float64)
        return (g64 / (1.0 + np.exp(-g64)) * u64).astype(np.float32)

    got = torch.full((n,), float("nan"), device=device)
    kk.gemv_kmajor_swiglu(x, wt, got, n, k, go, uo)
    assert_close(to_np(got), swiglu64(x_np), rtol=1e-4, atol=1e-5)
    # the two products and the activation as separate launches over the same stored weights
    both = torch.empty(2 * n, device=device)
    kk.gemv_kmajor(x, wt, both, 2 * n, k)
    sep = torch.empty(n, device=device)
    kk.swiglu(both[go:go + n].contiguous(), both[uo:uo + n].contiguous(), sep)
    assert_close(to_np(got), to_np(sep), rtol=1e-4, atol=1e-5)
    eps = 1e-5
    x64 = x_np.astype(np.float64)
    normed = (x64 / np.sqrt(np.mean(x64 * x64) + eps) * gamma_np).astype(np.float32)
    kk.gemv_kmajor_swiglu_normed(x, gamma, wt, got, n, k, go, uo, eps)
    assert_close(to_np(got), swiglu64(normed), rtol=1e-4, atol=1e-5)


# (m, k, widths): whole 128 x 96 tiles with split-K (q/k/v at 512 tokens); 128 x 64 tiles with
# split-K (o); 128 x 128 tiles; one member; partial tiles in m and n; K steps of 16; rows that take
# the B-streaming kernels (2..8) and the one-row kernel inside the grouped call
@pytest.mark.parametrize("m,k,widths", [
    (512, 2048, [2048, 512, 512]), (512, 2048, [2048]), (2048, 2048, [2048, 512, 512]), (512, 8192, [2048]),
    (1024, 512, [4096, 4096]), (200, 256, [1000]), (130, 72, [96, 40]), (4, 2048, [512, 64]),
    (1, 2048, [512, 64]), (9, 4096, [8]),
])
@pytest.mark.parametrize("storage", STORAGES)
def test_many_row_products_over_stored_weights_equal_fp32_over_the_widened(device, storage, m, k, widths):
    import torch
    kk = _k()
    total = sum(widths)
    rng = np.random.default_rng(m + k + total)
    a_np = rng.standard_normal((m, k), dtype=np.float32)
    wt, wide = _stored(rng.standard_normal((total, k), dtype=np.float32) * np.float32(0.05), storage, device)
    a, wide_dev = to_dev(a_np, device), to_dev(wide, device)
    got = [torch.full((m, w), float("nan"), device=device) for w in widths]
    kk.matmul_grouped(a, wt, got, m, k, widths, trans_b=True)
    exp = [torch.empty(m, w, device=device) for w in widths]
    kk.matmul_grouped(a, wide_dev, exp, m, k, widths, trans_b=True)
    off = 0
    for g, e, w in zip(got, exp, widths):
        assert_exact(to_np(g), to_np(e))
        e64 = a_np.astype(np.float64) @ wide[off:off + w].astype(np.float64).T
        assert_close(to_np(g), e64.astype(np.float32), rtol=1e-4, atol=1e-5 * np.sqrt(k))
        off += w


@pytest.mark.parametrize("m,n,k", [(512, 8192, 2048), (200, 16384, 64), (2048, 8192, 256)])
@pytest.mark.parametrize("storage", STORAGES)
def test_gate_up_swiglu_gemm_over_stored_weights_equals_fp32_over_the_widened(device, storage, m, n, k):
    import torch
    kk = _k()
    rng = np.random.default_rng(m + n + k)
    a_np = rng.standard_normal((m, k), dtype=np.float32)
    wt, wide = _stored(rng.standard_normal((2 * n, k), dtype=np.float32) * np.float32(0.05), storage, device)
    a, wide_dev = to_dev(a_np, device), to_dev(wide, device)
    for go, uo in ((0, n), (n, 0)):
        got = torch.full((m, n), float("nan"), device=device)
        kk.matmul_swiglu(a, wt, got, m, n, k, k, go, uo, trans_b=True)
        exp = torch.empty(m, n, device=device)
        kk.matmul_swiglu(a, wide_dev, exp, m, n, k, k, go, uo, trans_b=True)
        assert_exact(to_np(got), to_np(exp))


@pytest.mark.parametrize("storage", STORAGES)
def test_split_k_partials_over_stored_weights(device, storage):
    """The slabs a consumer adds up (rmlk_hip_matmul_partials) are those of the fp32 product."""
    import torch
    from rmlk_amd._lib import check, lib
    kk = _k()
    m, n, k = 512, 2048, 8192
    rng = np.random.default_rng(3)
    a = to_dev(rng.standard_normal((m, k), dtype=np.float32), device)
    wt, wide = _stored(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.05), storage, device)
    wide_dev = to_dev(wide, device)
    need = int(lib().rmlk_hip_matmul_partials_workspace_size(kk.FLOAT, m, n, k))
    stream = torch.cuda.current_stream().cuda_stream
    slabs = []
    for w in (wt, wide_dev):
        ws = torch.full((need // 4,), float("nan"), device=device)
        splits = ctypes.c_int32(0)
        check(lib().rmlk_hip_matmul_partials(stream, kk.FLOAT, m, n, k, a.data_ptr(), k, kk.storage_of(w),
                                             w.data_ptr(), k, 1, ws.data_ptr(), need, ctypes.byref(splits)),
              "rmlk_hip_matmul_partials")
        assert splits.value > 1
        slabs.append(to_np(ws[:splits.value * m * n]))
    assert_exact(slabs[0], slabs[1])


def test_stored_weights_argument_checks(device):
    import torch
    from rmlk_amd._lib import RmlkError
    kk = _k()
    n, k = 64, 256
    x = torch.randn(k, device=device)
    y = torch.empty(n, device=device)
    wt = kk.store_weights(torch.randn(n, k, device=device), torch.float16)
    a = torch.randn(16, k, device=device)
    out = [torch.empty(16, n, device=device)]
    with pytest.raises(RmlkError):          # 16-bit weights are K-contiguous only
        kk.matmul_grouped(a, wt, out, 16, k, [n], trans_b=False)
    with pytest.raises(RmlkError):          # rows of whole 128-bit units: k % 8
        kk.gemv_kmajor(x[:252], wt, y, n, 252)
    with pytest.raises(RmlkError):          # 16-byte aligned base
        kk.gemv_kmajor(x, wt.reshape(-1)[4:4 + (n - 1) * k], y, n - 1, k)
    with pytest.raises(RmlkError):          # int16 is not a storage type of weights
        kk.gemv_kmajor(x, wt.view(torch.int16), y, n, k)
    with pytest.raises(RmlkError):
        kk.store_weights(torch.randn(8, device=device), torch.int16)


# ---- sessions built with 16-bit weight storage ---------------------------------------------------

def _with_rounded_weights(graph, storage):
    """The same graph with every constant 2-D float matrix that is the second operand of a MatMul
    rounded to `storage` (and held as float32): what a session with that weight storage computes
    with."""
    from oracle import ops
    from rmlk_amd import runtime
    weights = {n.inputs[1] for n in graph.nodes if n.op == "MatMul" and len(n.inputs) == 2}
    gb = runtime.GraphBuilder()
    for name, (dt, dims) in graph.inputs.items():
        gb.input(name, dt, dims)
    for name, arr in graph.initializers.items():
        if name in weights and arr.ndim == 2 and arr.dtype == np.float32:
            arr = ops.store_weights(arr, storage)
        gb.constant(name, arr)
    for node in graph.nodes:
        ob = gb.op(node.op, [i or None for i in node.inputs], node.outputs)
        for key, value in node.attrs.items():
            ob.attr(key, value)
    for name in graph.outputs:
        gb.output(name)
    return gb.build()


@pytest.mark.parametrize("storage", STORAGES)
def test_decoder_layer_with_stored_weights_equals_fp32_over_rounded_weights(device, storage):
    """One full-width decoder layer, 256 tokens: every product is a tiled GEMM (joint q/k/v with its
    slabs left to the row streams, o and down with theirs left to the norm, gate/up with the SwiGLU
    epilogue) and those equal the fp32 kernels over the widened weights, so the outputs are EQUAL."""
    from oracle import graph as og
    from rmlk_amd import graphs, runtime
    graph, feeds = graphs.decoder_layer_graph(seed=3, seq=256)
    rounded = _with_rounded_weights(graph, storage)
    inst = runtime.Builder.from_graph(graph).build(0, weights=storage)
    ref = runtime.Builder.from_graph(rounded).build(0, weights="f32")
    assert inst.fused_nodes == ref.fused_nodes > 0
    got, exp = inst.run(feeds), ref.run(feeds)
    for name in exp:
        assert_exact(got[name], exp[name])
    # and the fp32 session on the ORIGINAL weights is a different (nearby) result: the storage is on
    full = runtime.Builder.from_graph(graph).build(0, weights="f32").run(feeds)
    first = next(iter(exp))
    assert not np.array_equal(full[first], got[first])
    oracle = og.run_graph(rounded, feeds)
    for name in oracle:
        assert_close(got[name], oracle[name], rtol=1e-3, atol=1e-4)
    inst.close()
    ref.close()


@pytest.mark.parametrize("storage", STORAGES)
@pytest.mark.parametrize("style", ["scatter", "concat"])
def test_llama_prefill_and_decode_with_stored_weights(device, storage, style):
    """Tiny Llama graph, prefill of 12 tokens and 4 greedy decode steps (one-row products, deferred
    norms, the projection inside the row streams): against the fp32 session over rounded weights and
    against the oracle walking that graph; same greedy tokens."""
    from oracle import graph as og
    from rmlk_amd import graphs, runtime
    cfg = graphs.LlamaConfig.tiny()
    max_len = 32
    graph = graphs.llama_graph(cfg, seed=4, style=style, max_len=max_len)
    rounded = _with_rounded_weights(graph, storage)
    inst = runtime.Builder.from_graph(graph).build(0, weights=storage)
    ref = runtime.Builder.from_graph(rounded).build(0, weights="f32")
    rng = np.random.default_rng(1)
    prompt = rng.integers(0, cfg.vocab, size=12)

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

    ids, past_len = prompt, 0
    outs = {"got": None, "ref": None, "oracle": None}
    for step in range(5):
        f = {name: feeds_for(ids, outs[name], past_len) for name in outs}
        outs["got"], outs["ref"] = inst.run(f["got"]), ref.run(f["ref"])
        outs["oracle"] = og.run_graph(rounded, f["oracle"])
        got, exp, orc = (outs[name]["logits"][0, -1] for name in ("got", "ref", "oracle"))
        assert_close(got, exp, rtol=1e-4, atol=1e-5)
        assert_close(got, orc, rtol=1e-3, atol=1e-4)
        tok = int(np.argmax(got))
        assert tok == int(np.argmax(exp)) == int(np.argmax(orc)), (step, tok)
        past_len += ids.size
        ids = np.array([tok])
    inst.close()
    ref.close()


def test_rows_that_are_no_whole_units_stay_float(device):
    """Weights whose K is no multiple of 8 are not stored as 16-bit values (their rows would not be
    whole 128-bit units): a session over such a graph gives the fp32 session's bits, and a graph
    that mixes both kinds what the fp32 session gives when only the storable weights are rounded."""
    from oracle import ops
    from rmlk_amd import graphs, runtime
    rng = np.random.default_rng(5)
    # hidden 60, ffn 100: no MatMul has K % 8 == 0
    cfg = graphs.LlamaConfig(layers=2, hidden=60, heads=15, kv_heads=3, head_dim=4, ffn=100, vocab=50)
    graph = graphs.llama_graph(cfg, seed=2, style="concat")
    feeds = graphs.llama_concat_inputs(cfg, rng.integers(0, cfg.vocab, size=9), None, 0)
    got = runtime.Builder.from_graph(graph).build(0, weights="bf16").run(feeds)
    exp = runtime.Builder.from_graph(graph).build(0).run(feeds)
    for name in exp:
        assert_exact(got[name], exp[name])
    # hidden 80 (storable), ffn 100 (the down projection stays float)
    cfg = graphs.LlamaConfig(layers=1, hidden=80, heads=20, kv_heads=4, head_dim=4, ffn=100, vocab=1000)
    graph = graphs.llama_graph(cfg, seed=3, style="concat")
    feeds = graphs.llama_concat_inputs(cfg, rng.integers(0, cfg.vocab, size=130), None, 0)
    weights = {n.inputs[1] for n in graph.nodes if n.op == "MatMul" and len(n.inputs) == 2}
    gb = runtime.GraphBuilder()
    for name, (dt, dims) in graph.inputs.items():
        gb.input(name, dt, dims)
    for name, arr in graph.initializers.items():
        if name in weights and arr.ndim == 2 and arr.shape[0] % 8 == 0:
            arr = ops.store_weights(arr, "f16")
        gb.constant(name, arr)
    for node in graph.nodes:
        ob = gb.op(node.op, [i or None for i in node.inputs], node.outputs)
        for key, value in node.attrs.items():
            ob.attr(key, value)
    for name in graph.outputs:
        gb.output(name)
    got = runtime.Builder.from_graph(graph).build(0, weights="f16").run(feeds)
    exp = runtime.Builder.from_graph(gb.build()).build(0, weights="f32").run(feeds)
    for name in exp:
        assert_exact(got[name], exp[name])


def test_weights_fit_tells_what_storage_would_change(device):
    import torch
    from oracle import ops
    kk = _k()
    rng = np.random.default_rng(8)
    w = (rng.standard_normal(100000) * 0.02).astype(np.float32)
    for storage, other in (("bf16", "f16"), ("f16", "bf16")):
        fitting = to_dev(ops.store_weights(w, storage), device)
        assert kk.weights_fit(fitting, _torch_dtype(storage))
        assert not kk.weights_fit(fitting, _torch_dtype(other))        # 8 against 11 significant bits, other ranges
        spoiled = fitting.clone()
        spoiled[77777] = float(np.nextafter(np.float32(0.02), np.float32(1)))
        assert not kk.weights_fit(spoiled, _torch_dtype(storage))
    assert not kk.weights_fit(to_dev(w, device), torch.bfloat16)
    special = to_dev(np.array([0.0, -0.0, np.inf, -np.inf, 1.0, -2.5], dtype=np.float32), device)
    assert kk.weights_fit(special, torch.bfloat16) and kk.weights_fit(special, torch.float16)
    assert not kk.weights_fit(to_dev(np.array([1.0, np.nan], dtype=np.float32), device), torch.bfloat16)
    assert kk.weights_fit(torch.empty(0, device=device), torch.float16)


@pytest.mark.parametrize("style", ["scatter", "concat"])
def test_weights_that_are_bfloat16_values_are_held_as_such(device, style):
    """A graph whose float weights are bfloat16 values already (a checkpoint trained in bfloat16): the
    session stores them in 16 bits without being asked, since nothing is lost. Against the session
    that keeps floats: the prefill (tiled products) bit for bit, decode steps to rounding, same
    tokens. Ordinary float weights stay floats."""
    from rmlk_amd import graphs, runtime
    cfg = graphs.LlamaConfig.tiny()
    max_len = 32
    graph = graphs.llama_graph(cfg, seed=4, style=style, max_len=max_len, bf16_values=True)
    auto = runtime.Builder.from_graph(graph).build(0)
    floats = runtime.Builder.from_graph(graph).build(0, weights="f32")
    assert auto.weights_16bit == 4 * cfg.layers + 1     # joint q/k/v, joint gate/up, o, down per layer; the lm-head
    assert floats.weights_16bit == 0
    plain = runtime.Builder.from_graph(graphs.llama_graph(cfg, seed=4, style=style, max_len=max_len)).build(0)
    assert plain.weights_16bit == 0
    plain.close()
    rng = np.random.default_rng(2)
    ids, past_len, outs = rng.integers(0, cfg.vocab, size=12), 0, {"auto": None, "floats": None}

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
        outs["auto"] = auto.run(feeds_for(ids, outs["auto"], past_len))
        outs["floats"] = floats.run(feeds_for(ids, outs["floats"], past_len))
        got, exp = outs["auto"]["logits"], outs["floats"]["logits"]
        if step == 0:
            assert_exact(got, exp)
        else:
            assert_close(got, exp, rtol=1e-4, atol=1e-5)
        tok = int(np.argmax(got[0, -1]))
        assert tok == int(np.argmax(exp[0, -1]))
        past_len += ids.size
        ids = np.array([tok])
    auto.close()
    floats.close()


def test_both_storage_flags_at_once_are_refused(device):
    from rmlk_amd import graphs, runtime
    from rmlk_amd._lib import lib
    graph = graphs.llama_graph(graphs.LlamaConfig.tiny(), seed=4, style="scatter", max_len=16)
    h = ctypes.c_void_p()
    for flags in (2 | 4, 2 | 8, 4 | 8):
        assert lib().rmlk_session_create_ex(graph.handle, 0, flags, ctypes.byref(h)) != 0
        assert not h

"""Whole-graph parity on the GPU: the benchmark configurations (rmlk_amd.graphs) through the native
executor against the CPU oracle walking the same graph.

Bars: fp32 outputs within rtol 1e-4 / atol 1e-5 per op-sized graph (config 1, 3), logits within
the reference's Llama e2e bar (atol = rtol = 1e-2, runtime/tests/e2e_ort/cases.rs:80-81) and
identical greedy tokens for the Llama graphs; integer / move outputs bit-exact (config 5).
No reference-held vectors exist for the Llama graphs and ONNX Runtime is not installable here:
whole-graph parity is against the numpy oracle only (parity unpinned beyond the per-op pins)."""
import os

import numpy as np
import pytest

from helpers import assert_close, assert_exact

pytestmark = pytest.mark.gpu


def _rt():
    from rmlk_amd import graphs, runtime
    return graphs, runtime


def _oracle():
    from oracle import graph as og
    return og


def test_attention_fixture_through_runtime(device):
    """runtime/tests/graphs/attention.rs:8-56 against the ONNX-Runtime-generated fixture."""
    _, runtime = _rt()
    here = os.path.dirname(os.path.abspath(__file__))
    q, k, v = (np.fromfile(os.path.join(here, "golden", f"attention_{n}.f32"), dtype="<f4")
               .reshape(1, 2, 4) for n in "qkv")
    exp = np.fromfile(os.path.join(here, "golden", "attention_out.f32"), dtype="<f4")
    g = runtime.GraphBuilder()
    for n in "qkv":
        g.input(n, np.float32, [1, 2, 4])
    g.constant("scale", np.array(2.0, dtype=np.float32))
    g.op("Transpose", ["k"], ["kt"]).attr("perm", [0, 2, 1])
    g.op("MatMul", ["q", "kt"], ["scores"])
    g.op("Div", ["scores", "scale"], ["scaled"])
    g.op("Trilu", ["scaled"], ["masked"]).attr("upper", 0)
    g.op("Softmax", ["masked"], ["probs"]).attr("axis", -1)
    g.op("MatMul", ["probs", "v"], ["out"])
    g.output("out")
    inst = runtime.Builder.from_graph(g.build()).build()
    out = inst.run({"q": q, "k": k, "v": v})["out"]
    np.testing.assert_allclose(out.reshape(-1), exp, rtol=0, atol=1e-5)
    assert inst.memory_stats()["device_syncs"] == 0


def test_config1_rmsnorm_matmul(device):
    graphs, runtime = _rt()
    graph, feeds = graphs.rmsnorm_matmul_graph(seed=1)
    inst = runtime.Builder.from_graph(graph).build()
    got = inst.run(feeds)["y"]
    exp = _oracle().run_graph(graph, feeds)["y"]
    assert got.shape == (1, 128, 8192)
    assert_close(got, exp, rtol=1e-4, atol=1e-5)


def test_config3_decoder_layer_small_seq(device):
    """Full-width layer (hidden 2048, 32/8 heads, FFN 8192) at a sequence the CPU oracle finishes
    in seconds; the S = 2048 shape runs in the properties test below."""
    graphs, runtime = _rt()
    graph, feeds = graphs.decoder_layer_graph(seed=3, seq=96)
    inst = runtime.Builder.from_graph(graph).build()
    got = inst.run(feeds)["y"]
    exp = _oracle().run_graph(graph, feeds)["y"]
    assert_close(got, exp, rtol=1e-4, atol=2e-5)
    assert inst.memory_stats()["device_syncs"] == 0  # shape chains resolved on the host


def test_config3_full_sequence_properties(device):
    """S = 2048: causality (output row i does not depend on later tokens) and determinism."""
    graphs, runtime = _rt()
    graph, feeds = graphs.decoder_layer_graph(seed=3, seq=2048)
    inst = runtime.Builder.from_graph(graph).build()
    y = inst.run(feeds)["y"]
    assert y.shape == (1, 2048, 2048) and np.isfinite(y).all()
    x2 = feeds["x"].copy()
    x2[:, 1500:] += 1.0
    y2 = inst.run({"x": x2})["y"]
    assert_exact(y2[:, :1500], y[:, :1500])
    assert np.abs(y2[:, 1500:] - y[:, 1500:]).max() > 1e-3
    # the first 96 rows of the long run equal the short run (same weights, causal attention)
    graph_s, feeds_s = graphs.decoder_layer_graph(seed=3, seq=96)
    exp = _oracle().run_graph(graph_s, {"x": feeds["x"][:, :96]})["y"]
    assert_close(y[:, :96], exp, rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("fuse", [True, False], ids=["fused", "one_kernel_per_node"])
def test_config3_full_sequence_every_row_against_the_oracle(device, fuse):
    """S = 2048, the sequence length the configuration names: every one of the 2048 output rows of
    the layer against the oracle walking the same graph (fp32 BLAS, one [1,32,2048,2048] softmax:
    seconds on the host). With fusion this is where the resident-grid attention kernel that skips
    hidden key chunks and the 128 x 192 q/k/v tiles run; without it, one kernel per node as the
    reference executes a graph. The bar of the short-sequence test: rtol 1e-4 / atol 2e-5
    (multi-op graphs in the reference: abs 1e-5 at toy sizes, runtime/tests/graphs/main.rs:28-40)."""
    graphs, runtime = _rt()
    graph, feeds = graphs.decoder_layer_graph(seed=3, seq=2048)
    exp = _oracle().run_graph(graph, feeds, "f32")["y"]
    inst = runtime.Builder.from_graph(graph).build(fuse=fuse)
    try:
        assert (inst.fused_nodes > 0) == fuse
        got = inst.run(feeds)["y"]
    finally:
        inst.close()
    assert got.shape == exp.shape == (1, 2048, 2048)
    assert_close(got, exp, rtol=1e-4, atol=2e-5)


def _greedy_concat(inst, graphs, cfg, prompt, steps):
    feeds = graphs.llama_concat_inputs(cfg, prompt, None, 0)
    out = inst.run(feeds)
    logits = [out["logits"][0, -1].copy()]
    toks = [int(np.argmax(logits[-1]))]
    past_len = prompt.size
    for _ in range(steps - 1):
        feeds = graphs.llama_concat_inputs(cfg, np.array([toks[-1]]), out, past_len)
        out = inst.run(feeds)
        logits.append(out["logits"][0, -1].copy())
        toks.append(int(np.argmax(logits[-1])))
        past_len += 1
    return toks, logits


def test_llama_tiny_concat_style_vs_oracle(device):
    """The reference's I/O contract (zero-length caches on step 0, cache grown by Concat)."""
    graphs, runtime = _rt()
    cfg = graphs.LlamaConfig.tiny()
    graph = graphs.llama_graph(cfg, seed=4, style="concat")
    inst = runtime.Builder.from_graph(graph).build()
    rng = np.random.default_rng(4)
    prompt = rng.integers(0, cfg.vocab, size=12)
    toks, logits = _greedy_concat(inst, graphs, cfg, prompt, 5)

    og = _oracle()
    feeds = graphs.llama_concat_inputs(cfg, prompt, None, 0)
    out = og.run_graph(graph, feeds)
    past_len = prompt.size
    for step in range(5):
        ref = out["logits"][0, -1]
        np.testing.assert_allclose(logits[step], ref, rtol=1e-2, atol=1e-2)
        assert_close(logits[step], ref.astype(np.float32), rtol=1e-3, atol=1e-4)
        assert int(np.argmax(ref)) == toks[step]          # teacher-forced, like e2e_ort/llama.rs
        feeds = graphs.llama_concat_inputs(cfg, np.array([toks[step]]), out, past_len)
        out = og.run_graph(graph, feeds)
        past_len += 1
    assert inst.memory_stats()["device_syncs"] == 0


def _scatter_feeds(cfg, ids, start, caches):
    s = ids.size
    feeds = {"input_ids": ids.reshape(1, s).astype(np.int64),
             "position_ids": np.arange(start, start + s, dtype=np.int64).reshape(1, s)}
    feeds.update(caches)
    return feeds


def test_llama_tiny_scatter_style_equals_concat_style(device):
    """Fixed-length caches + ScatterND give the same logits and tokens as the growing caches; the
    recorded HIP graph of a decode step replays to the same results as eager steps."""
    graphs, runtime = _rt()
    cfg = graphs.LlamaConfig.tiny()
    max_len = 32
    gc = graphs.llama_graph(cfg, seed=4, style="concat")
    gs = graphs.llama_graph(cfg, seed=4, style="scatter", max_len=max_len)
    rng = np.random.default_rng(5)
    prompt = rng.integers(0, cfg.vocab, size=9)
    steps = 6
    ic = runtime.Builder.from_graph(gc).build()
    toks_c, logits_c = _greedy_concat(ic, graphs, cfg, prompt, steps)

    zeros = {f"cache.{l}.{kv}": np.zeros((1, cfg.kv_heads, max_len, cfg.head_dim), np.float32)
             for l in range(cfg.layers) for kv in ("key", "value")}

    def run_scatter(use_graph):
        inst = runtime.Builder.from_graph(gs).build()
        out = inst.run(_scatter_feeds(cfg, prompt, 0, zeros))
        logits = [out["logits"][0, -1].copy()]
        toks = [int(np.argmax(logits[-1]))]
        pos = prompt.size
        captured = False
        for _ in range(steps - 1):
            inst.set_input("input_ids", np.array([[toks[-1]]], dtype=np.int64))
            inst.set_input("position_ids", np.array([[pos]], dtype=np.int64))
            if not captured:
                for l in range(cfg.layers):
                    for kv in ("key", "value"):
                        inst.feed_output(f"cache_out.{l}.{kv}", f"cache.{l}.{kv}")
            if use_graph:
                if not captured:
                    inst.capture()
                    captured = True
                inst.replay()
            else:
                inst.execute()
                captured = False
            lg = inst.output("logits")[0, -1].copy()
            logits.append(lg)
            toks.append(int(np.argmax(lg)))
            pos += 1
        stats = inst.memory_stats()
        inst.close()
        return toks, logits, stats

    toks_e, logits_e, stats_e = run_scatter(False)
    toks_g, logits_g, stats_g = run_scatter(True)
    assert toks_e == toks_c and toks_g == toks_c
    for a, b_, c in zip(logits_c, logits_e, logits_g):
        assert_close(b_, a, rtol=1e-4, atol=1e-5)
        assert_exact(c, b_)      # replay runs the same kernels on the same data
    assert stats_e["device_syncs"] == 0 and stats_g["device_syncs"] == 0


@pytest.mark.timeout(900)
@pytest.mark.parametrize("bf16_values,bf16_pieces", [(False, False), (True, False), (True, True)])
def test_llama_1b_full_size_prefill_and_teacher_forced_decode(device, bf16_values, bf16_pieces):
    """(bf16_values: the same graph with weights that are bfloat16 values held as floats, which the
    session stores in 16 bits by itself: the products over stored weights at the full widths -
    lm-head over 128256 rows, gate / up / down at 8192 - against the oracle on the same graph.
    bf16_pieces: the prefill's products on the bf16 matrix cores, the fp32 operand as three exact
    bfloat16 pieces - every one of the 65 products, none of the decode steps'.)

    BASELINE configs[3] at its full size: 16 layers, hidden 2048, vocab 128256. Prefill of a
    512-token prompt, then 8 decode steps through the recorded HIP graph with the caches fed back on
    the device, each step teacher-forced with the oracle's token and held to the reference's bar for
    whole-model runs (logits atol = rtol = 1e-2, identical argmax: runtime/tests/e2e_ort/llama.rs:112-156,
    cases.rs:75-85). The oracle multiplies in fp32 BLAS here (its float64 products would take minutes
    at this size); no ONNX Runtime vectors exist for this graph (parity unpinned beyond the oracle)."""
    graphs, runtime = _rt()
    og = _oracle()
    cfg = graphs.LlamaConfig()
    prompt_len, steps = 512, 8
    max_len = prompt_len + steps
    graph = graphs.llama_graph(cfg, seed=4, style="scatter", max_len=max_len, bf16_values=bf16_values)
    rng = np.random.default_rng(4)
    prompt = rng.integers(0, cfg.vocab, size=prompt_len)
    zeros = {f"cache.{l}.{kv}": np.zeros((1, cfg.kv_heads, max_len, cfg.head_dim), np.float32)
             for l in range(cfg.layers) for kv in ("key", "value")}
    inst = runtime.Builder.from_graph(graph).build(bf16_pieces=bf16_pieces)
    assert inst.weights_16bit == (4 * cfg.layers + 1 if bf16_values else 0)
    feeds = _scatter_feeds(cfg, prompt, 0, zeros)
    for name, arr in feeds.items():
        inst.set_input(name, arr)
    inst.execute()
    assert inst.products_bf16_pieces == (4 * cfg.layers + 1 if bf16_pieces else 0)
    got = inst.output("logits")[0, -1].copy()
    exp = og.run_graph(graph, feeds, matmul_accumulate="f32")
    pos = prompt_len
    captured = False
    for step in range(steps + 1):
        ref = exp["logits"][0, -1]
        np.testing.assert_allclose(got, ref, rtol=1e-2, atol=1e-2, err_msg=f"step {step}")
        tok = int(np.argmax(ref))
        assert int(np.argmax(got)) == tok, f"step {step}"
        if step == steps:
            break
        caches = {f"cache.{l}.{kv}": exp[f"cache_out.{l}.{kv}"] for l in range(cfg.layers)
                  for kv in ("key", "value")}
        exp = og.run_graph(graph, _scatter_feeds(cfg, np.array([tok]), pos, caches), matmul_accumulate="f32")
        inst.set_input("input_ids", np.array([[tok]], dtype=np.int64))
        inst.set_input("position_ids", np.array([[pos]], dtype=np.int64))
        if not captured:
            for l in range(cfg.layers):
                for kv in ("key", "value"):
                    inst.feed_output(f"cache_out.{l}.{kv}", f"cache.{l}.{kv}")
            inst.capture()
            captured = True
        inst.replay()
        got = inst.output("logits")[0, -1].copy()
        pos += 1
    assert inst.memory_stats()["device_syncs"] == 0
    assert inst.products_bf16_pieces == 0      # (one-row products stream their weights as before)
    inst.close()


@pytest.mark.parametrize("heads,kv_heads,head_dim,hidden,ffn", [
    (6, 2, 64, 384, 640),      # head_dim 64: the attention kernels and the row-stream launch run
    (4, 2, 128, 512, 768),     # head_dim 128: the attention chain falls back to its three kernels
    (3, 3, 64, 192, 260),      # no grouped-query repeat, widths that are no multiple of a tile
])
def test_llama_other_widths_scatter_style_vs_oracle(device, heads, kv_heads, head_dim, hidden, ffn):
    """Prefill of 70 tokens and four decode steps (caches fed back on the device) of Llama-shaped
    graphs of other widths against the oracle, teacher-forced like e2e_ort/llama.rs."""
    graphs, runtime = _rt()
    og = _oracle()
    cfg = graphs.LlamaConfig(layers=2, hidden=hidden, heads=heads, kv_heads=kv_heads, head_dim=head_dim,
                             ffn=ffn, vocab=1000)
    max_len = 100
    graph = graphs.llama_graph(cfg, seed=7, style="scatter", max_len=max_len)
    rng = np.random.default_rng(7)
    prompt = rng.integers(0, cfg.vocab, size=70)
    zeros = {f"cache.{l}.{kv}": np.zeros((1, cfg.kv_heads, max_len, cfg.head_dim), np.float32)
             for l in range(cfg.layers) for kv in ("key", "value")}
    inst = runtime.Builder.from_graph(graph).build()
    got = inst.run(_scatter_feeds(cfg, prompt, 0, zeros))
    exp = og.run_graph(graph, _scatter_feeds(cfg, prompt, 0, zeros))
    assert_close(got["logits"], exp["logits"], rtol=1e-3, atol=1e-4)
    for l in range(cfg.layers):
        for kv in ("key", "value"):
            assert_close(got[f"cache_out.{l}.{kv}"], exp[f"cache_out.{l}.{kv}"], rtol=1e-3, atol=1e-4)
    pos = prompt.size
    for _ in range(4):
        tok = int(np.argmax(exp["logits"][0, -1]))
        assert int(np.argmax(got["logits"][0, -1])) == tok
        caches = {f"cache.{l}.{kv}": exp[f"cache_out.{l}.{kv}"] for l in range(cfg.layers)
                  for kv in ("key", "value")}
        exp = og.run_graph(graph, _scatter_feeds(cfg, np.array([tok]), pos, caches))
        inst.set_input("input_ids", np.array([[tok]], dtype=np.int64))
        inst.set_input("position_ids", np.array([[pos]], dtype=np.int64))
        for l in range(cfg.layers):        # the caches stay on the device, updated in place
            for kv in ("key", "value"):
                inst.feed_output(f"cache_out.{l}.{kv}", f"cache.{l}.{kv}")
        inst.execute()
        got = {"logits": inst.output("logits")}
        assert_close(got["logits"], exp["logits"], rtol=1e-3, atol=1e-4)
        pos += 1
    assert inst.memory_stats()["device_syncs"] == 0
    inst.close()


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_llama_shapes_with_and_without_fusion(device, seed):
    """Llama-shaped graphs of random widths, head counts, sequence and cache lengths, both cache
    styles: the session with pattern fusion agrees with the one-kernel-per-node session, and gives
    the same bits when it runs again on recycled buffers."""
    graphs, runtime = _rt()
    rng = np.random.default_rng(seed)
    for _ in range(8):
        head_dim = int(rng.choice([4, 8, 16, 64, 64, 128]))
        kv_heads = int(rng.choice([1, 2, 3, 4]))
        heads = kv_heads * int(rng.choice([1, 2, 4, 5]))
        hidden = heads * head_dim
        if hidden > 2048:
            continue
        vocab = int(rng.choice([50, 300, 1000]))
        style = str(rng.choice(["scatter", "concat"]))
        seq = int(rng.choice([1, 2, 3, 7, 16, 33, 64, 70, 130]))
        max_len = -(-(seq + int(rng.integers(1, 40))) // 4) * 4
        cfg = graphs.LlamaConfig(layers=int(rng.choice([1, 2])), hidden=hidden, heads=heads, kv_heads=kv_heads,
                                 head_dim=head_dim, ffn=int(rng.choice([64, 100, 256, 520])), vocab=vocab)
        case = f"{cfg} {style} seq={seq} max_len={max_len}"
        if style == "scatter":
            graph = graphs.llama_graph(cfg, seed=seed, style="scatter", max_len=max_len)
            feeds = {"input_ids": rng.integers(0, vocab, size=(1, seq)).astype(np.int64),
                     "position_ids": np.arange(seq, dtype=np.int64).reshape(1, seq)}
            for l in range(cfg.layers):
                for kv in ("key", "value"):
                    feeds[f"cache.{l}.{kv}"] = (rng.standard_normal((1, kv_heads, max_len, head_dim),
                                                                    dtype=np.float32) * np.float32(0.1))
        else:
            graph = graphs.llama_graph(cfg, seed=seed, style="concat")
            feeds = graphs.llama_concat_inputs(cfg, rng.integers(0, vocab, size=seq), None, 0)
        fused = runtime.Builder.from_graph(graph).build(fuse=True)
        plain = runtime.Builder.from_graph(graph).build(fuse=False)
        a, b, again = fused.run(feeds), plain.run(feeds), fused.run(feeds)
        for name in a:
            np.testing.assert_allclose(a[name], b[name], rtol=2e-3, atol=2e-4, err_msg=f"{name} of {case}")
            assert np.array_equal(a[name], again[name], equal_nan=True), f"{name} of {case} is not repeatable"
        fused.close()
        plain.close()


def test_config5_kv_stress_small_vs_oracle(device):
    graphs, runtime = _rt()
    graph, feeds = graphs.kv_stress_graph(seed=5, length=256, vocab=1000, hidden=128,
                                          n_gather=77, mask_n=96)
    inst = runtime.Builder.from_graph(graph).build()
    got = inst.run(feeds)
    exp = _oracle().run_graph(graph, feeds)
    for name in graph.outputs:
        assert_exact(got[name], np.asarray(exp[name]))


def test_config5_kv_stress_full_size_properties(device):
    """Full sizes of config 5 checked through properties numpy states directly (no oracle walk of
    the 1 GB table): scatter touches exactly one row per head, grow = slice ++ row, gather rows
    equal table rows, masks equal triu / comparisons of index grids."""
    graphs, runtime = _rt()
    graph, feeds = graphs.kv_stress_graph(seed=5)
    inst = runtime.Builder.from_graph(graph).build()
    got = inst.run(feeds)
    cache, row, idx = feeds["cache"], feeds["row"], feeds["scatter_idx"]
    pos = int(idx[0, 0, 0, 2])
    exp = cache.copy()
    exp[0, :, pos, :] = row[0, :, 0, :]
    assert_exact(got["scattered"], exp)
    assert_exact(got["grown"], np.concatenate([cache[:, :, :-1], row], axis=2))
    table = graph.initializers[[n for n in graph.initializers if n.startswith("table")][0]]
    assert_exact(got["gathered"], table[feeds["gather_idx"]])
    assert_exact(got["tri"], np.triu(feeds["tri_in"], 1))
    n = feeds["rows"].shape[0]
    assert got["mask_gt"].dtype == np.bool_ and got["mask_gt"].shape == (n, n)
    assert_exact(got["mask_gt"], np.triu(np.ones((n, n), bool), 1))
    assert_exact(got["mask_eq"], np.eye(n, dtype=bool))

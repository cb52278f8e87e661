"""Synthetic ONNX-operator graphs of the benchmark configurations (random-init weights, seeded).

Built with GraphBuilder out of exactly the operators of the reference's Llama path
(runtime/src/providers/cuda/backend/mod.rs:82-162): no fused operators, RMSNorm is
Pow -> ReduceMean -> Add -> Sqrt -> Div -> Mul, SwiGLU is Sigmoid / Mul / Mul, attention is
MatMul / Div / Add(mask) / Softmax / MatMul, RoPE goes through Cast / Mul / Concat / Sin / Cos and
Slice / Neg / Concat, GQA through Unsqueeze / Expand / Reshape.

Two Llama graph styles:
  * "concat": the I/O contract of the reference's example (runtime/examples/llama.rs:62-161):
    input_ids, attention_mask, position_ids, past_key_values.{l}.{key,value} [1, KV, past, D] ->
    logits, present.{l}.{key,value}; the cache grows by Concat, the mask comes from Trilu / Where.
  * "scatter": fixed-length caches cache.{l}.{key,value} [1, KV, MAX, D] updated by ScatterND at
    position_ids, mask from Range / Greater / Where. Shapes do not depend on the step, so a decode
    step can be recorded once into a HIP graph and replayed.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from .runtime import Graph, GraphBuilder

FLOAT, INT64, BOOL = 1, 7, 9


@dataclass
class LlamaConfig:
    """Llama-3.2-1B shape by default (16 layers, hidden 2048, 32 query / 8 KV heads of 64)."""
    layers: int = 16
    hidden: int = 2048
    heads: int = 32
    kv_heads: int = 8
    head_dim: int = 64
    ffn: int = 8192
    vocab: int = 128256
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5

    @staticmethod
    def tiny(layers=2):
        return LlamaConfig(layers=layers, hidden=128, heads=8, kv_heads=2, head_dim=16, ffn=256,
                           vocab=500)


class _B:
    """GraphBuilder with generated value names."""

    def __init__(self):
        self.g = GraphBuilder()
        self.n = 0
        self.consts = {}

    def name(self, hint):
        self.n += 1
        return f"{hint}_{self.n}"

    def op(self, op, inputs, hint=None, out=None, **attrs):
        out = out or self.name(hint or op.lower())
        ob = self.g.op(op, inputs, [out])
        for k, v in attrs.items():
            ob.attr(k, v)
        return out

    def const(self, arr, hint="c"):
        arr = np.asarray(arr)
        key = (arr.dtype.str, arr.shape, arr.tobytes()) if arr.size <= 64 else None
        if key is not None and key in self.consts:
            return self.consts[key]
        name = self.name(hint)
        self.g.constant(name, arr)
        if key is not None:
            self.consts[key] = name
        return name

    def i64(self, vals):
        return self.const(np.array(vals, dtype=np.int64), "i")

    def f32(self, val):
        return self.const(np.array(val, dtype=np.float32), "f")


def _rmsnorm(b: _B, x, gamma, eps):
    """Decomposed RMSNorm: x -> Pow(2) -> ReduceMean(-1, keepdims) -> Add(eps) -> Sqrt ->
    Div(x, .) -> Mul(gamma)."""
    sq = b.op("Pow", [x, b.f32(2.0)], "rms_pow")
    mean = b.op("ReduceMean", [sq], "rms_mean", axes=[-1], keepdims=1)
    var = b.op("Add", [mean, b.f32(eps)], "rms_add")
    rms = b.op("Sqrt", [var], "rms_sqrt")
    normed = b.op("Div", [x, rms], "rms_div")
    return b.op("Mul", [normed, gamma], "rms_mul")


def rmsnorm_matmul_graph(seed=1, seq=128, hidden=2048, n_out=8192):
    """Config 1: decomposed RMSNorm followed by MatMul with W.
    x [1,seq,hidden] ~ N(0,1) is the graph input; gamma ~ U(0.5,1.5); W ~ N(0,0.02)."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((1, seq, hidden), dtype=np.float32)
    gamma = rng.uniform(0.5, 1.5, size=(hidden,)).astype(np.float32)
    w = (rng.standard_normal((hidden, n_out), dtype=np.float32) * np.float32(0.02))
    b = _B()
    b.g.input("x", FLOAT, [1, seq, hidden])
    g_name = b.const(gamma, "gamma")
    w_name = b.const(w, "W")
    y = _rmsnorm(b, "x", g_name, 1e-5)
    b.op("MatMul", [y, w_name], out="y")
    b.g.output("y")
    return b.g.build(), {"x": x}


def as_bfloat16_values(x: np.ndarray) -> np.ndarray:
    """x (float32) rounded to the nearest bfloat16 value, ties to even, still float32: weights as a
    checkpoint trained in bfloat16 and exported as float holds them."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return (u & 0xFFFFFFFF).astype(np.uint32).view(np.float32).reshape(x.shape)


def _weights(rng, cfg: LlamaConfig, layer: int, bf16_values: bool = False):
    def w(shape):
        x = rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02)
        return as_bfloat16_values(x) if bf16_values else x
    h, kvd = cfg.hidden, cfg.kv_heads * cfg.head_dim
    return {
        "ln1": np.ones((h,), np.float32), "ln2": np.ones((h,), np.float32),
        "wq": w((h, cfg.heads * cfg.head_dim)), "wk": w((h, kvd)), "wv": w((h, kvd)),
        "wo": w((cfg.heads * cfg.head_dim, h)),
        "wg": w((h, cfg.ffn)), "wu": w((h, cfg.ffn)), "wd": w((cfg.ffn, h)),
    }


def _rope_tables(b: _B, cfg: LlamaConfig, position_ids):
    """cos / sin [1,1,S,D] from position_ids [1,S] (int64) and the inverse-frequency table."""
    half = cfg.head_dim // 2
    inv_freq = (1.0 / (cfg.rope_theta ** (np.arange(0, half, dtype=np.float64) * 2 / cfg.head_dim)))
    inv = b.const(inv_freq.astype(np.float32).reshape(1, 1, half), "inv_freq")
    pos_f = b.op("Cast", [position_ids], "pos_f", to=FLOAT)              # [1,S]
    pos_3 = b.op("Unsqueeze", [pos_f, b.i64([2])], "pos_3")              # [1,S,1]
    freqs = b.op("Mul", [pos_3, inv], "freqs")                           # [1,S,half]
    emb = b.op("Concat", [freqs, freqs], "rope_emb", axis=-1)            # [1,S,D]
    cos = b.op("Unsqueeze", [b.op("Cos", [emb], "cos"), b.i64([1])], "cos4")   # [1,1,S,D]
    sin = b.op("Unsqueeze", [b.op("Sin", [emb], "sin"), b.i64([1])], "sin4")
    return cos, sin


def _rotate_half(b: _B, x, cfg: LlamaConfig):
    half = cfg.head_dim // 2
    x1 = b.op("Slice", [x, b.i64([0]), b.i64([half]), b.i64([3])], "rot_x1")
    x2 = b.op("Slice", [x, b.i64([half]), b.i64([cfg.head_dim]), b.i64([3])], "rot_x2")
    return b.op("Concat", [b.op("Neg", [x2], "rot_neg"), x1], "rot_cat", axis=-1)


def _apply_rope(b: _B, x, cos, sin, cfg):
    a = b.op("Mul", [x, cos], "rope_xc")
    r = b.op("Mul", [_rotate_half(b, x, cfg), sin], "rope_rs")
    return b.op("Add", [a, r], "rope")


def _split_heads(b: _B, x, n_heads, cfg):
    """[1,S,n*D] -> [1,n,S,D]"""
    r = b.op("Reshape", [x, b.i64([1, -1, n_heads, cfg.head_dim])], "heads_rs")
    return b.op("Transpose", [r], "heads_tr", perm=[0, 2, 1, 3])


def _repeat_kv(b: _B, x, cfg):
    """GQA: [1,KV,L,D] -> [1,H,L,D] via Unsqueeze / Expand / Reshape."""
    rep = cfg.heads // cfg.kv_heads
    if rep == 1:
        return x
    u = b.op("Unsqueeze", [x, b.i64([2])], "gqa_u")                      # [1,KV,1,L,D]
    e = b.op("Expand", [u, b.i64([1, cfg.kv_heads, rep, 1, 1])], "gqa_e")   # [1,KV,rep,L,D]
    return b.op("Reshape", [e, b.i64([1, cfg.heads, -1, cfg.head_dim])], "gqa_r")


def _attention(b: _B, q, k_all, v_all, mask, cfg):
    kx = _repeat_kv(b, k_all, cfg)
    vx = _repeat_kv(b, v_all, cfg)
    kt = b.op("Transpose", [kx], "k_t", perm=[0, 1, 3, 2])                # [1,H,D,L]
    scores = b.op("MatMul", [q, kt], "scores")                           # [1,H,S,L]
    scaled = b.op("Div", [scores, b.f32(float(np.sqrt(cfg.head_dim)))], "scaled")
    masked = b.op("Add", [scaled, mask], "masked")
    probs = b.op("Softmax", [masked], "probs", axis=-1)
    ctx = b.op("MatMul", [probs, vx], "ctx")                             # [1,H,S,D]
    ctx_t = b.op("Transpose", [ctx], "ctx_t", perm=[0, 2, 1, 3])          # [1,S,H,D]
    return b.op("Reshape", [ctx_t, b.i64([1, -1, cfg.heads * cfg.head_dim])], "ctx_r")


def _mlp(b: _B, x, wn):
    gate = b.op("MatMul", [x, wn["wg"]], "gate")
    up = b.op("MatMul", [x, wn["wu"]], "up")
    silu = b.op("Mul", [gate, b.op("Sigmoid", [gate], "sig")], "silu")    # x * sigmoid(x)
    act = b.op("Mul", [silu, up], "act")
    return b.op("MatMul", [act, wn["wd"]], "down")


def _layer(b: _B, x, wn, cfg, cos, sin, kv_update, mask):
    """One decoder layer. kv_update(k_new, v_new) -> (k_all, v_all) applies the cache policy."""
    h1 = _rmsnorm(b, x, wn["ln1"], cfg.rms_eps)
    q = _split_heads(b, b.op("MatMul", [h1, wn["wq"]], "q"), cfg.heads, cfg)
    k = _split_heads(b, b.op("MatMul", [h1, wn["wk"]], "k"), cfg.kv_heads, cfg)
    v = _split_heads(b, b.op("MatMul", [h1, wn["wv"]], "v"), cfg.kv_heads, cfg)
    q = _apply_rope(b, q, cos, sin, cfg)
    k = _apply_rope(b, k, cos, sin, cfg)
    k_all, v_all = kv_update(k, v)
    attn = _attention(b, q, k_all, v_all, mask, cfg)
    x = b.op("Add", [x, b.op("MatMul", [attn, wn["wo"]], "o")], "res1")
    h2 = _rmsnorm(b, x, wn["ln2"], cfg.rms_eps)
    return b.op("Add", [x, _mlp(b, h2, wn)], "res2")


def _layer_consts(b: _B, w, l):
    return {k: b.const(v, f"l{l}_{k}") for k, v in w.items()}


def _causal_mask_trilu(b: _B, scores_like_q, k_len_source, past_len_1d):
    """[1,1,S,L] additive mask: Trilu(upper, k = past + 1) of a -inf matrix shaped from the run-time
    S and L, as exported Llama graphs build it (Shape / Gather / Concat / ConstantOfShape / Trilu)."""
    s = b.op("Gather", [b.op("Shape", [scores_like_q], "shp_q"), b.i64([2])], "s_len")      # [1]
    l = b.op("Gather", [b.op("Shape", [k_len_source], "shp_k"), b.i64([2])], "l_len")       # [1]
    shape2 = b.op("Concat", [s, l], "mask_shape", axis=0)
    neg = b.op("ConstantOfShape", [shape2], "mask_fill",
               value=np.array([-np.inf], dtype=np.float32))
    k = b.op("Add", [past_len_1d, b.i64([1])], "mask_k")
    k0 = b.op("Reshape", [k, b.const(np.zeros((0,), np.int64), "empty_shape")], "mask_k0")  # scalar
    tri = b.op("Trilu", [neg, k0], "mask_tri", upper=1)
    return b.op("Unsqueeze", [tri, b.i64([0, 1])], "mask4")


def decoder_layer_graph(seed=3, seq=2048, cfg: LlamaConfig | None = None, bf16_values=False):
    """Config 3: one Llama-3.2-1B-shaped decoder layer, prefill at batch 1 (token embeddings
    ~ N(0,1) are the graph input `x` [1,S,hidden]; no cache). bf16_values: every weight a bfloat16
    value held as float (see as_bfloat16_values)."""
    cfg = cfg or LlamaConfig()
    rng = np.random.default_rng(seed)
    w = _weights(rng, cfg, 0, bf16_values)
    x = rng.standard_normal((1, seq, cfg.hidden), dtype=np.float32)
    b = _B()
    b.g.input("x", FLOAT, [1, 0, cfg.hidden])
    wn = _layer_consts(b, w, 0)
    # positions 0..S-1 from Range over the run-time sequence length
    s_len = b.op("Gather", [b.op("Shape", ["x"], "x_shape"), b.i64([1])], "seq_len")        # [1]
    s0 = b.op("Reshape", [s_len, b.const(np.zeros((0,), np.int64), "empty_shape")], "seq_len0")
    pos = b.op("Range", [b.const(np.array(0, np.int64)), s0, b.const(np.array(1, np.int64))], "pos")
    pos2 = b.op("Unsqueeze", [pos, b.i64([0])], "pos2")                                     # [1,S]
    cos, sin = _rope_tables(b, cfg, pos2)
    state = {}

    def kv_update(k, v):
        state["k"] = k
        return k, v

    # mask needs a [.., S, ..] and a [.., L, ..] source; here L == S, taken from the rotated k
    def layer_with_mask():
        h1 = _rmsnorm(b, "x", wn["ln1"], cfg.rms_eps)
        q = _split_heads(b, b.op("MatMul", [h1, wn["wq"]], "q"), cfg.heads, cfg)
        k = _split_heads(b, b.op("MatMul", [h1, wn["wk"]], "k"), cfg.kv_heads, cfg)
        v = _split_heads(b, b.op("MatMul", [h1, wn["wv"]], "v"), cfg.kv_heads, cfg)
        q = _apply_rope(b, q, cos, sin, cfg)
        k = _apply_rope(b, k, cos, sin, cfg)
        mask = _causal_mask_trilu(b, q, k, b.i64([0]))
        attn = _attention(b, q, k, v, mask, cfg)
        x1 = b.op("Add", ["x", b.op("MatMul", [attn, wn["wo"]], "o")], "res1")
        h2 = _rmsnorm(b, x1, wn["ln2"], cfg.rms_eps)
        return b.op("Add", [x1, _mlp(b, h2, wn)], out="y")

    layer_with_mask()
    b.g.output("y")
    return b.g.build(), {"x": x}


def llama_graph(cfg: LlamaConfig | None = None, seed=4, style="scatter", max_len=640, bf16_values=False):
    """Config 4: the full Llama-shaped graph (tied embedding: Gather on `embed`, final MatMul with
    the same values laid out [hidden, vocab]). Returns the Graph; inputs are built by the callers
    (llama_inputs_*)."""
    cfg = cfg or LlamaConfig()
    rng = np.random.default_rng(seed)
    b = _B()
    embed = rng.standard_normal((cfg.vocab, cfg.hidden), dtype=np.float32) * np.float32(0.02)
    if bf16_values:     # every weight a bfloat16 value held as float (see as_bfloat16_values)
        embed = as_bfloat16_values(embed)
    embed_n = b.const(embed, "embed")
    lm_head_n = b.const(np.ascontiguousarray(embed.T), "lm_head")
    del embed
    final_ln = b.const(np.ones((cfg.hidden,), np.float32), "final_ln")
    b.g.input("input_ids", INT64, [1, 0])
    b.g.input("position_ids", INT64, [1, 0])
    if style == "concat":
        b.g.input("attention_mask", INT64, [1, 0])
        for l in range(cfg.layers):
            for kv in ("key", "value"):
                b.g.input(f"past_key_values.{l}.{kv}", FLOAT, [1, cfg.kv_heads, 0, cfg.head_dim])
    else:
        for l in range(cfg.layers):
            for kv in ("key", "value"):
                b.g.input(f"cache.{l}.{kv}", FLOAT, [1, cfg.kv_heads, max_len, cfg.head_dim])
    x = b.op("Gather", [embed_n, "input_ids"], "tok_embed", axis=0)               # [1,S,hidden]
    cos, sin = _rope_tables(b, cfg, "position_ids")

    if style == "concat":
        # past length from the cache shape; causal part from Trilu, padding part from
        # attention_mask through Equal / Where
        past_len = b.op("Gather", [b.op("Shape", ["past_key_values.0.key"], "past_shape"),
                                   b.i64([2])], "past_len")                     # [1]
        total_mask = b.op("Unsqueeze", ["attention_mask", b.i64([1, 2])], "am4")  # [1,1,1,L]
        pad = b.op("Equal", [total_mask, b.const(np.array(0, np.int64))], "am_is_pad")
    else:
        # scatter indices [1,KV,S,3] = (0, head, position) and the step-independent mask
        pos4 = b.op("Unsqueeze", ["position_ids", b.i64([1, 3])], "pos4")         # [1,1,S,1]
        pos_e = b.op("Expand", [pos4, b.i64([1, cfg.kv_heads, 1, 1])], "pos_e")   # [1,KV,S,1]
        heads = b.const(np.arange(cfg.kv_heads, dtype=np.int64).reshape(1, cfg.kv_heads, 1, 1),
                        "head_ids")
        head_e = b.op("Add", [b.op("Mul", [pos_e, b.const(np.array(0, np.int64))], "zeros_i"),
                              heads], "head_e")                                   # [1,KV,S,1]
        zero_e = b.op("Mul", [pos_e, b.const(np.array(0, np.int64))], "batch_e")
        scatter_idx = b.op("Concat", [zero_e, head_e, pos_e], "scatter_idx", axis=-1)
        key_pos = b.op("Range", [b.const(np.array(0, np.int64)), b.const(np.array(max_len, np.int64)),
                                 b.const(np.array(1, np.int64))], "key_pos")        # [MAX]
        future = b.op("Greater", [key_pos, pos4], "future")                       # [1,1,S,MAX]
        mask = b.op("Where", [future, b.f32(-np.inf), b.f32(0.0)], "mask")

    outputs = []
    for l in range(cfg.layers):
        wn = _layer_consts(b, _weights(rng, cfg, l, bf16_values), l)
        if style == "concat":
            def kv_update(k, v, l=l):
                k_all = b.op("Concat", [f"past_key_values.{l}.key", k], out=f"present.{l}.key", axis=2)
                v_all = b.op("Concat", [f"past_key_values.{l}.value", v], out=f"present.{l}.value",
                             axis=2)
                return k_all, v_all
            if l == 0:
                # the mask needs q and k_all of the first layer for its run-time shape
                h1 = _rmsnorm(b, x, wn["ln1"], cfg.rms_eps)
                q = _split_heads(b, b.op("MatMul", [h1, wn["wq"]], "q"), cfg.heads, cfg)
                k = _split_heads(b, b.op("MatMul", [h1, wn["wk"]], "k"), cfg.kv_heads, cfg)
                v = _split_heads(b, b.op("MatMul", [h1, wn["wv"]], "v"), cfg.kv_heads, cfg)
                q = _apply_rope(b, q, cos, sin, cfg)
                k = _apply_rope(b, k, cos, sin, cfg)
                k_all, v_all = kv_update(k, v)
                causal = _causal_mask_trilu(b, q, k_all, past_len)
                mask = b.op("Where", [pad, b.f32(-np.inf), causal], "mask")
                attn = _attention(b, q, k_all, v_all, mask, cfg)
                x = b.op("Add", [x, b.op("MatMul", [attn, wn["wo"]], "o")], "res1")
                h2 = _rmsnorm(b, x, wn["ln2"], cfg.rms_eps)
                x = b.op("Add", [x, _mlp(b, h2, wn)], "res2")
            else:
                x = _layer(b, x, wn, cfg, cos, sin, kv_update, mask)
            outputs += [f"present.{l}.key", f"present.{l}.value"]
        else:
            def kv_update(k, v, l=l):
                k_all = b.op("ScatterND", [f"cache.{l}.key", scatter_idx, k],
                             out=f"cache_out.{l}.key")
                v_all = b.op("ScatterND", [f"cache.{l}.value", scatter_idx, v],
                             out=f"cache_out.{l}.value")
                return k_all, v_all
            x = _layer(b, x, wn, cfg, cos, sin, kv_update, mask)
            outputs += [f"cache_out.{l}.key", f"cache_out.{l}.value"]
    hf = _rmsnorm(b, x, final_ln, cfg.rms_eps)
    b.op("MatMul", [hf, lm_head_n], out="logits")
    b.g.output("logits")
    for o in outputs:
        b.g.output(o)
    return b.g.build()


def llama_concat_inputs(cfg: LlamaConfig, ids: np.ndarray, past: dict | None, past_len: int):
    """Feeds of the concat-style graph for a chunk of token ids after `past_len` cached tokens
    (zero-length caches on the first step, runtime/examples/llama.rs:17-20)."""
    s = ids.size
    feeds = {
        "input_ids": ids.reshape(1, s).astype(np.int64),
        "position_ids": np.arange(past_len, past_len + s, dtype=np.int64).reshape(1, s),
        "attention_mask": np.ones((1, past_len + s), dtype=np.int64),
    }
    for l in range(cfg.layers):
        for kv in ("key", "value"):
            name = f"past_key_values.{l}.{kv}"
            feeds[name] = (past[f"present.{l}.{kv}"] if past is not None else
                           np.zeros((1, cfg.kv_heads, 0, cfg.head_dim), np.float32))
    return feeds


def kv_stress_graph(seed=5, heads=8, length=8192, head_dim=64, vocab=128256, hidden=2048,
                    n_gather=4096, mask_n=8192):
    """Config 5: indexing / KV-cache stress, every integer path bit-exact.
    ScatterND writes one new token row [1,H,1,D] into a cache [1,H,L,D] at a random position;
    Slice shrinks the cache by one row and Concat grows it back to L with the new row; Gather
    takes n_gather rows of a [vocab, hidden] table; Trilu(upper, k=1) and Equal / Greater build
    boolean masks over [mask_n, mask_n]."""
    rng = np.random.default_rng(seed)
    cache = rng.standard_normal((1, heads, length, head_dim), dtype=np.float32)
    row = rng.standard_normal((1, heads, 1, head_dim), dtype=np.float32)
    pos = int(rng.integers(0, length))
    idx = np.array([[[[0, h, pos]] for h in range(heads)]], dtype=np.int64)   # [1,H,1,3]
    table = rng.standard_normal((vocab, hidden), dtype=np.float32)
    gidx = rng.integers(0, vocab, size=(n_gather,), dtype=np.int64)
    tri_in = rng.standard_normal((mask_n, mask_n), dtype=np.float32)
    rows = np.arange(mask_n, dtype=np.int64).reshape(mask_n, 1)
    cols = np.arange(mask_n, dtype=np.int64).reshape(1, mask_n)
    b = _B()
    b.g.input("cache", FLOAT, list(cache.shape))
    b.g.input("row", FLOAT, list(row.shape))
    b.g.input("scatter_idx", INT64, list(idx.shape))
    b.g.input("gather_idx", INT64, [n_gather])
    b.g.input("tri_in", FLOAT, [mask_n, mask_n])
    b.g.input("rows", INT64, [mask_n, 1])
    b.g.input("cols", INT64, [1, mask_n])
    table_n = b.const(table, "table")
    b.op("ScatterND", ["cache", "scatter_idx", "row"], out="scattered")
    head = b.op("Slice", ["cache", b.i64([0]), b.i64([length - 1]), b.i64([2])], "kv_head")
    b.op("Concat", [head, "row"], out="grown", axis=2)
    b.op("Gather", [table_n, "gather_idx"], out="gathered", axis=0)
    b.op("Trilu", ["tri_in", b.const(np.array(1, np.int64))], out="tri", upper=1)
    b.op("Greater", ["cols", "rows"], out="mask_gt")
    b.op("Equal", ["cols", "rows"], out="mask_eq")
    for o in ("scattered", "grown", "gathered", "tri", "mask_gt", "mask_eq"):
        b.g.output(o)
    feeds = {"cache": cache, "row": row, "scatter_idx": idx, "gather_idx": gidx, "tri_in": tri_in,
             "rows": rows, "cols": cols}
    return b.g.build(), feeds

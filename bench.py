#!/usr/bin/env python3
"""Benchmark of the operator path on one MI355X.

Default workload (BASELINE.json configs[3], the configuration the headline metric is quoted on):
the full Llama-3.2-1B-shaped fp32 graph (16 layers, hidden 2048, 32/8 heads of 64, FFN 8192,
vocab 128256, random-init weights ~ N(0, 0.02), synthetic token ids), fixed-length KV caches
updated by ScatterND. One "step" is one prefill pass over a 512-token prompt; after the timed
prefill steps, 128 greedy decode steps are timed as well (a decode step is one replay of the
recorded HIP graph plus the host argmax over the logits).

Prints ONE JSON line: value = prefill tokens/s (inputs resident in HBM, K steps timed between
stream synchronisations), plus decode ms/token, the roofline of the dominant kernel (fp32 MFMA
GEMM) measured with HIP events, and the CPU oracle timed on the host cores on a bounded sample.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--prompt 512] [--decode 128]
    python bench.py --suite ops        # per-kernel launches of the op microbench shapes (for rocprofv3)
    python bench.py --suite c1|c3|c5   # BASELINE configs[0], [2], [4] as graphs, fused and one kernel per node
    python bench.py --summarize-ops JSON --kernel-trace CSV [--pmc-fetch CSV --pmc-write CSV]
    python bench.py --summarize-graph JSON --kernel-trace CSV
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0   # dense bf16 MFMA
PEAK_HBM_GBS = 8000.0
CALIBRATION_COPY_BYTES = 256 << 20

# HBM-side traffic of one GEMM launch per shape (batch, m, n, k[, epilogue]) of the default workload:
# (kernel the library chose when the counters were read, KiB fetched, KiB written). RECORDED values,
# not measured by the run that prints them: read with `rocprofv3 --pmc FETCH_SIZE` and `--pmc
# WRITE_SIZE` (one run each) over `python3 bench.py --no-cpu --steps 1 --warmup 0 --decode 4`, scaled
# by what the same counters read for the 256 MiB calibration copy below (FETCH_SIZE 131092 -> x2.0,
# WRITE_SIZE 262144 -> x1.0); summary and command in PMC_TRAFFIC_SOURCE. An entry counts only while
# the library still picks the kernel named with it. Split-K launches write partial sums to the
# workspace; what their consumer (the combine kernel or the norm kernel) moves is not included.
PMC_TRAFFIC_SOURCE = "profiles/gemm_mfma_llama1b_prefill512_hbm_traffic.md"
PMC_TRAFFIC_KIB = {
    (1, 512, 3072, 2048): ("mfma128x96x32 direct splitk=2", 41142, 12288),                # q/k/v
    (1, 512, 2048, 2048): ("mfma128x64x32 direct splitk=4", 24709, 16384),                # o
    (1, 512, 2048, 8192): ("mfma128x64x32 direct splitk=4", 130473, 16384),                # down
    (1, 512, 16384, 2048, "swiglu"): ("mfma128x128x32 direct splitk=1", 207740, 16384),   # gate/up, SwiGLU epilogue
    (1, 512, 128256, 2048): ("mfma128x128x32 direct splitk=1", 1844647, 256512),          # lm-head
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def cpu_threads():
    """(threads the oracle's BLAS products run on, a description of the BLAS pool)."""
    try:
        from threadpoolctl import threadpool_info
        pools = [p for p in threadpool_info() if p.get("user_api") == "blas"]
        if pools:
            n = max(int(p["num_threads"]) for p in pools)
            return n, ", ".join(f"{p.get('internal_api', '?')} x{p['num_threads']}" for p in pools)
    except Exception:           # threadpoolctl missing or numpy not loaded yet: fall back to the environment
        pass
    n = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return n, f"OMP_NUM_THREADS / cpu_count = {n}"


def cpu_baseline(graph, cfg, graphs, prompt, n_tokens, max_len):
    """The numpy oracle (fp32 BLAS matmuls) on the host: prefill of the first n_tokens of the same
    prompt through the same graph."""
    import numpy as np
    from oracle import graph as og
    prompt = prompt[:n_tokens]
    feeds = {"input_ids": prompt.reshape(1, -1).astype(np.int64),
             "position_ids": np.arange(n_tokens, dtype=np.int64).reshape(1, -1)}
    for l in range(cfg.layers):
        for kv in ("key", "value"):
            feeds[f"cache.{l}.{kv}"] = np.zeros((1, cfg.kv_heads, max_len, cfg.head_dim), np.float32)
    t0 = time.perf_counter()
    out = og.run_graph(graph, feeds, matmul_accumulate="f32")
    dt = time.perf_counter() - t0
    return n_tokens / dt, dt, out["logits"][0, -1]


def run_llama(args):
    import numpy as np
    import torch
    from rmlk_amd import graphs, kernels, runtime

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    info = kernels.device_info(0)
    cfg = graphs.LlamaConfig() if not args.tiny else graphs.LlamaConfig.tiny()
    prompt_len, decode_steps = args.prompt, args.decode
    max_len = prompt_len + decode_steps
    t0 = time.perf_counter()
    graph = graphs.llama_graph(cfg, seed=4, style="scatter", max_len=max_len, bf16_values=args.bf16_values)
    log(f"[bench] graph built in {time.perf_counter() - t0:.1f}s: {len(graph.nodes)} nodes")
    t0 = time.perf_counter()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(0)[0]
    inst = runtime.Builder.from_graph(graph).build(0, weights=args.weights, bf16_pieces=args.bf16_pieces)
    torch.cuda.synchronize()
    weights_resident = free_before - torch.cuda.mem_get_info(0)[0]
    # how the session ended up holding the weights: as asked, or ("auto") 16-bit where nothing is lost
    stored = args.weights if args.weights in ("f16", "bf16") else ("bf16" if inst.weights_16bit else "f32")
    log(f"[bench] session created (weights uploaded) in {time.perf_counter() - t0:.1f}s, "
        f"{weights_resident / 1e9:.2f} GB of device memory")

    # A plain copy of known size (256 MiB read + 256 MiB written by copy_flat_kernel): the unit
    # that rocprofv3's FETCH_SIZE / WRITE_SIZE readings of the other kernels are scaled by.
    calib = torch.empty(2 * CALIBRATION_COPY_BYTES // 4, dtype=torch.float32, device="cuda:0")
    n_cal = CALIBRATION_COPY_BYTES // 4
    kernels.concat_into(calib[:n_cal], calib[n_cal:], [n_cal], [n_cal], 0, 0)
    torch.cuda.synchronize()
    del calib

    rng = np.random.default_rng(4)
    prompt = rng.integers(0, cfg.vocab, size=prompt_len)
    caches = {f"cache.{l}.{kv}": np.zeros((1, cfg.kv_heads, max_len, cfg.head_dim), np.float32)
              for l in range(cfg.layers) for kv in ("key", "value")}

    def feed_prefill():
        inst.set_input("input_ids", prompt.reshape(1, -1).astype(np.int64))
        inst.set_input("position_ids", np.arange(prompt_len, dtype=np.int64).reshape(1, -1))
        for name, arr in caches.items():
            inst.set_input(name, arr)

    # ---- prefill: warm-up, then K timed steps (replays of the recorded graph) ------------------
    feed_prefill()
    inst.execute()                       # first run: fills the buffer pool
    first_logits = inst.output("logits")[0, -1].copy()
    prefill_products_bf16 = inst.products_bf16_pieces
    inst.capture()
    for _ in range(args.warmup):
        inst.replay()
    inst.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        inst.replay_enqueue()            # the passes queue up behind one another: no host round trip between them
    inst.check()                         # waits for all of them; a kernel failure of any pass is reported here
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    ms_per_step = prefill_s / args.steps * 1e3
    tok_s = prompt_len * args.steps / prefill_s
    replay_logits = inst.output("logits")[0, -1].copy()
    assert np.array_equal(first_logits, replay_logits), "replayed prefill differs from the eager run"
    mem = inst.memory_stats()
    mem["session_device_bytes_after_build"] = int(weights_resident)
    log(f"[bench] prefill {prompt_len} tokens: {ms_per_step:.2f} ms/step, {tok_s:.0f} tok/s")

    # ---- roofline of the MatMul kernels: one extra eager pass with HIP events per node ----------
    feed_prefill()
    inst.set_profiling(True)
    inst.execute()
    inst.set_profiling(False)
    stats = inst.node_stats()
    # classify each MatMul node by the kernel the library picks for its shape
    launches = matmul_launches(cfg, prompt_len, max_len)
    mm_nodes = [s for s in stats if s["op"] in ("MatMul", "rmlk.MatMulGroup", "rmlk.MatMulGroupSwiGLU",
                                                "rmlk.MatMulAddRMSNorm", "rmlk.MatMulConst")]
    assert len(mm_nodes) == len(launches), (len(mm_nodes), len(launches))
    by_kind, per_op = {}, {}
    for s, shapes in zip(mm_nodes, launches):
        node_flops = sum(2.0 * sh[0] * sh[1] * sh[2] * sh[3] for sh in shapes)
        for shape in shapes:
            batch, m, n, k = shape[:4]
            swiglu = len(shape) > 4        # n counts the gate and the up columns; n / 2 are written
            kind = kernels.matmul_describe(batch, m, n, k)
            d = by_kind.setdefault(kind, {"launches": 0, "us": 0.0, "flops": 0.0, "alg_bytes": 0.0,
                                          "traffic": 0.0, "shapes": {}})
            d["launches"] += 1
            d["shapes"][shape] = d["shapes"].get(shape, 0) + 1
            flops = 2.0 * batch * m * n * k
            d["us"] += s["micros"] * flops / node_flops     # a node of several launches: by flops
            d["flops"] += flops
            w_bytes = 4.0 if stored == "f32" else 2.0
            d["alg_bytes"] += batch * (4.0 * m * k + w_bytes * k * n + 4.0 * m * (n // 2 if swiglu else n))
            pmc = PMC_TRAFFIC_KIB.get(shape) if stored == "f32" else None
            if pmc is not None and pmc[0] != kind:
                pmc = None                       # another kernel than the one the counters were read for
            d["traffic"] = None if pmc is None or d["traffic"] is None else d["traffic"] + 1024.0 * sum(pmc[1:])
    for s in stats:
        if s["micros"] > 0:
            d = per_op.setdefault(s["op"], {"n": 0, "us": 0.0, "bytes": 0.0})
            d["n"] += 1
            d["us"] += s["micros"]
            d["bytes"] += s["bytes"]
    eager_us = sum(d["us"] for d in per_op.values())
    dom_kind = max(by_kind, key=lambda kd: by_kind[kd]["us"])
    dom = by_kind[dom_kind]
    # The dominant kernel's launch duration: the launches it makes in one prefill pass (same shapes,
    # same counts, weights rotated so that they come from HBM as in the model), issued back to back
    # through the C ABI between ONE pair of HIP events on the stream they run on. (The per-node
    # events above add a cache write-back after every node, ~10 us on a 16 MiB output.)
    pieces = bool(prefill_products_bf16)   # the products ran as bfloat16 pieces on the bf16 matrix cores
    dom_us = time_matmul_launches(kernels, torch, dom["shapes"], storage=stored, pieces=pieces)
    achieved = dom["flops"] / dom["launches"] / (dom_us * 1e-6) / 1e12
    roofline = {
        "bound": "mfma",
        "kernel": f"{'gemm_mfma_direct_kernel' if 'direct' in dom_kind else 'gemm_mfma_kernel'} ({dom_kind})",
        "achieved": round(achieved, 2), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
        "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
        "traffic": None if dom["traffic"] is None else round(dom["traffic"] / dom["launches"]),
        "traffic_unit": "HBM bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, copy-calibrated)",
        "traffic_source": f"recorded table from {PMC_TRAFFIC_SOURCE} (an earlier counter run of this command), "
                          "not measured by this run; null when the library picks another kernel than then",
        "algorithmic_bytes_per_launch": round(dom["alg_bytes"] / dom["launches"]),
        "launches": dom["launches"], "avg_launch_us": round(dom_us, 2),
        "avg_node_us_with_events": round(dom["us"] / dom["launches"], 2),
        "flops_per_launch": dom["flops"] / dom["launches"],
        "shapes": {"x".join(map(str, k_[:4])) + ("".join(" " + t for t in k_[4:])): v
                   for k_, v in dom["shapes"].items()},
        "measured": "one HIP event pair around the kernel's launches of one prefill pass (same shapes "
                    "and counts, cold weights), 4 repetitions after 8 untimed ones, on the launching stream",
    }
    if pieces:
        # three bf16 MFMAs per product: priced against the bf16 peak at three times the fp32 flops
        roofline.update({
            "kernel": f"gemm_bf16x3_kernel (the launches that the fp32 path would give to: {dom_kind})",
            "achieved": round(3 * achieved, 2), "peak": PEAK_BF16_MFMA_TFLOPS,
            "frac": round(3 * achieved / PEAK_BF16_MFMA_TFLOPS, 4),
            "fp32_equivalent_tflops": round(achieved, 2), "traffic": None,
            "flops_per_launch": 3 * dom["flops"] / dom["launches"],
            "note": "bf16 flops = 3 x 2 M N K (hi, mid and lo piece of the fp32 operand); the split of the "
                    "operand into pieces is a launch of its own and not part of this duration"})
    all_mm_flops = sum(d["flops"] for d in by_kind.values())
    all_mm_us = sum(d["us"] for d in by_kind.values())
    matmul_all = {"tflops": round(all_mm_flops / (all_mm_us * 1e-6) / 1e12, 2),
                  "frac_of_fp32_mfma_peak": round(all_mm_flops / (all_mm_us * 1e-6) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                  "share_of_prefill_time": round(all_mm_us / eager_us, 3),
                  "by_kernel": {k_: {"launches": v["launches"], "us": round(v["us"], 1),
                                     "tflops": round(v["flops"] / (v["us"] * 1e-6) / 1e12, 2)}
                                for k_, v in by_kind.items()}}
    op_breakdown = {op: {"n": d["n"], "us": round(d["us"], 1),
                         "gbs": round(d["bytes"] / (d["us"] * 1e-6) / 1e9, 1) if d["us"] > 0 else 0}
                    for op, d in sorted(per_op.items(), key=lambda kv: -kv[1]["us"])}

    # ---- decode: recorded HIP graph of one step, replayed decode_steps times -------------------
    decode_ms, tokens = None, []
    if decode_steps > 0:
        for l in range(cfg.layers):
            for kv in ("key", "value"):
                inst.feed_output(f"cache_out.{l}.{kv}", f"cache.{l}.{kv}")
        tok = int(np.argmax(first_logits))
        pos = prompt_len
        inst.set_input("input_ids", np.array([[tok]], dtype=np.int64))
        inst.set_input("position_ids", np.array([[pos]], dtype=np.int64))
        inst.capture()
        logits_buf = np.empty((1, 1, cfg.vocab), dtype=np.float32)
        inst.sync()
        t0 = time.perf_counter()
        for _ in range(decode_steps):
            inst.set_input("input_ids", np.array([[tok]], dtype=np.int64))
            inst.set_input("position_ids", np.array([[pos]], dtype=np.int64))
            inst.replay()
            tok = int(np.argmax(inst.output("logits")))
            tokens.append(tok)
            pos += 1
        inst.sync()
        decode_ms = (time.perf_counter() - t0) / decode_steps * 1e3
        # device-only time of a step: replays without the host round trip
        inst.sync()
        t0 = time.perf_counter()
        for _ in range(20):
            inst.replay_enqueue()
        inst.check()
        decode_dev_ms = (time.perf_counter() - t0) / 20 * 1e3
        weight_bytes = decode_weight_bytes(cfg, stored)
        log(f"[bench] decode: {decode_ms:.3f} ms/token end to end, {decode_dev_ms:.3f} ms/token "
            f"device replay ({weight_bytes / decode_dev_ms / 1e6:.0f} GB/s of weights)")
    else:
        decode_dev_ms, weight_bytes = None, decode_weight_bytes(cfg, stored)

    # ---- CPU baseline: the oracle on a bounded sample -------------------------------------------
    cpu = None
    if not args.no_cpu and args.weights in ("f32", "auto"):
        n_cpu = min(args.cpu_tokens, prompt_len)
        cores, blas = cpu_threads()
        cpu_tok_s, cpu_s, cpu_logits = cpu_baseline(graph, cfg, graphs, prompt, n_cpu, max_len)
        # the same sample through the GPU session (eager), as a check of the measured path
        inst.set_input("input_ids", prompt[:n_cpu].reshape(1, -1).astype(np.int64))
        inst.set_input("position_ids", np.arange(n_cpu, dtype=np.int64).reshape(1, -1))
        for name, arr in caches.items():
            inst.set_input(name, arr)
        inst.execute()
        gpu_logits = inst.output("logits")[0, -1]
        diff = float(np.max(np.abs(gpu_logits - cpu_logits)))
        same_top1 = int(np.argmax(gpu_logits)) == int(np.argmax(cpu_logits))
        assert diff <= 1e-2 and same_top1, f"GPU and oracle disagree on the sample: {diff}, top-1 {same_top1}"
        cpu = {"value": round(cpu_tok_s, 2), "unit": "tok/s", "cores": cores,
               "kind": "port",
               "sample": f"prefill of the first {n_cpu} prompt tokens through the same graph with the "
                         f"numpy oracle (fp32 BLAS matmuls, {blas}), {cpu_s:.1f} s; "
                         "ONNX Runtime is not installed",
               "gpu_vs_oracle_on_sample": {"max_abs_logit_diff": round(diff, 6), "top1_equal": same_top1,
                                           "bar": "1e-2 on logits, identical top-1"}}
        log(f"[bench] cpu oracle: {cpu_tok_s:.1f} tok/s over {n_cpu} tokens ({cpu_s:.1f}s); "
            f"GPU logits of the sample within {diff:.2e}, top-1 equal: {same_top1}")

    result = {
        "metric": "llama3.2-1b-shape fp32 prefill tok/s (decode ms/tok alongside)",
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if not prefill_products_bf16 else "f32 (many-row products: exact products of bf16 pieces, f32 accumulation)",
        "data": "synthetic",
        "weight_storage": stored, "weight_storage_asked": args.weights,
        "weights_are_bfloat16_values": bool(args.bf16_values),
        "prefill_products_on_bf16_matrix_cores": prefill_products_bf16,
        "config": {"workload": "BASELINE configs[3]: full Llama-3.2-1B-shaped ONNX-op graph, fp32, "
                               f"prefill {prompt_len} tokens + {decode_steps} greedy decode steps, batch 1, "
                               "KV cache updated by ScatterND, random-init weights N(0,0.02)",
                   "layers": cfg.layers, "hidden": cfg.hidden, "vocab": cfg.vocab,
                   "prompt_tokens": prompt_len, "graph_nodes": len(graph.nodes),
                   "execution": "recorded HIP graph replay per step; the timed replays are enqueued back to back and awaited once"},
        "decode_ms_per_token": None if decode_ms is None else round(decode_ms, 4),
        "decode_device_ms_per_token": None if decode_dev_ms is None else round(decode_dev_ms, 4),
        "decode_weight_gbs": None if decode_dev_ms is None else round(weight_bytes / decode_dev_ms / 1e6, 1),
        "decode_frac_of_hbm_peak": None if decode_dev_ms is None else round(weight_bytes / decode_dev_ms / 1e6 / PEAK_HBM_GBS, 4),
        "roofline": roofline, "matmul_all": matmul_all, "ops": op_breakdown,
        "cpu_baseline": cpu,
        "memory": mem, "device": info["name"], "arch": info["arch"],
    }
    inst.close()
    return result


def time_matmul_launches(kernels, torch, shape_counts, reps=4, warm_reps=8, storage="f32", pieces=False):
    """Average duration (us) of rmlk_hip_matmul launches: for every (batch, m, n, k) -> count, `count`
    launches with a broadcast 2-D K-contiguous weight operand taken in turn from enough distinct buffers to
    exceed the 256 MB Infinity Cache, all between one pair of HIP events on the current stream.
    `warm_reps` untimed repetitions come first: after the event-per-node pass (idle gaps) the chip
    needs some tens of milliseconds of continuous work before launch durations settle at what the
    replayed model sees (304 -> 271 -> 259 -> 249 -> ~240 us per repetition on the gate/up launch)."""
    dev = torch.device("cuda:0")
    plans, total = [], 0
    for shape, count in shape_counts.items():
        batch, m, n, k = shape[:4]
        swiglu = len(shape) > 4
        a = torch.randn(batch, m, k, device=dev)
        nb = max(2, min(count, int(600e6 // (4 * k * n)) + 1))
        bs = [torch.randn(n, k, device=dev) * 0.02 for _ in range(nb)]   # K-contiguous, as a session stores weights
        if storage != "f32":
            bs = [kernels.store_weights(b, {"f16": torch.float16, "bf16": torch.bfloat16}[storage]) for b in bs]
        c = torch.empty(batch, m, n // 2 if swiglu else n, device=dev)
        need = kernels.matmul_workspace_size(batch, m, n, k)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
        # pieces: the launches of rmlk_hip_matmul_bf16x3 over the operand split beforehand
        a3 = kernels.bf16x3_split(a[0]) if pieces else None
        plans.append((batch, m, n, k, swiglu, count, a, bs, c, ws, a3))
        total += count

    def run_once():
        for batch, m, n, k, swiglu, count, a, bs, c, ws, a3 in plans:
            for i in range(count):
                if pieces and swiglu:
                    kernels.matmul_bf16x3_swiglu(a3, bs[i % len(bs)], c, m, n // 2, k, 0, n // 2)
                elif pieces:
                    kernels.matmul_bf16x3(a3, bs[i % len(bs)], c, m, n, k)
                elif swiglu:
                    kernels.matmul_swiglu(a, bs[i % len(bs)], c, m, n // 2, k, k, 0, n // 2, trans_b=True)
                elif storage != "f32":
                    # (the product over stored weights: the grouped entry point with one member)
                    kernels.matmul_grouped(a, bs[i % len(bs)], [c], m, k, [n], workspace=ws, trans_b=True)
                else:
                    kernels.matmul(a, bs[i % len(bs)], c, batch, m, n, k, k, k, n, m * k, 0, m * n,
                                   trans_b=True, workspace=ws)
    for _ in range(warm_reps):
        run_once()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        run_once()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (reps * total)


def decode_weight_bytes(cfg, storage="f32"):
    """Weights streamed once per decoded token: per layer q,o,k,v,gate,up,down + lm-head, 4 bytes
    each as the reference holds them, 2 with 16-bit weight storage."""
    kvd = cfg.kv_heads * cfg.head_dim
    per_layer = (2 * cfg.hidden * cfg.heads * cfg.head_dim + 2 * cfg.hidden * kvd +
                 3 * cfg.hidden * cfg.ffn)
    return (4.0 if storage == "f32" else 2.0) * (cfg.layers * per_layer + cfg.hidden * cfg.vocab)


def matmul_launches(cfg, s, max_len):
    """(batch, m, n, k[, "swiglu"]) of the GEMM launches behind every MatMul-type node of the fused
    scatter-style graph, in node order: q/k/v (one node, one launch over the joint weights), o,
    gate/up (one node, one launch with the SwiGLU epilogue; n counts both halves), down per layer,
    then the lm-head. (Scores, softmax and context are one attention kernel, not a GEMM launch.)"""
    h, kvd, d = cfg.hidden, cfg.kv_heads * cfg.head_dim, cfg.head_dim
    whole = s % 128 == 0 and h % 128 == 0 and kvd % 128 == 0 and cfg.ffn % 64 == 0
    qkv = [(1, s, cfg.heads * d + 2 * kvd, h)] if whole else \
        [(1, s, cfg.heads * d, h), (1, s, kvd, h), (1, s, kvd, h)]
    gate_up = [(1, s, 2 * cfg.ffn, h, "swiglu")] if cfg.ffn % 64 == 0 and h % 32 == 0 and s >= 128 and \
        ((s + 127) // 128) * (cfg.ffn // 64) >= 256 else \
        [(1, s, cfg.ffn, h), (1, s, cfg.ffn, h)]
    out = []
    for _ in range(cfg.layers):
        out += [qkv, [(1, s, h, cfg.heads * d)], gate_up, [(1, s, h, cfg.ffn)]]
    out.append([(1, s, cfg.vocab, h)])
    return out


def run_ops_suite(args):
    """BASELINE configs[1] and configs[4] operator shapes, each launched repeatedly over rotating buffer
    sets (working set well above the 256 MB Infinity Cache, so that HBM is what is measured).
    A one-block `write_small_kernel` launch marks the start of every op in a kernel trace:
    `bench.py --summarize-ops` splits a `rocprofv3 --kernel-trace` (and `--pmc`) CSV of this command
    at those markers."""
    import ctypes
    import numpy as np
    import torch
    from rmlk_amd import kernels as k
    from rmlk_amd._lib import check, lib
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(2)
    ns = 16                             # 16 x 33.5 MB per operand
    shp, n = [8, 32, 512, 64], 8 * 32 * 512 * 64
    xs = [torch.randn(n, device=dev, generator=g) for _ in range(ns)]
    ys = [torch.empty(n, device=dev) for _ in range(ns)]
    bs = [torch.randn(32 * 64, device=dev, generator=g) for _ in range(ns)]
    conds = [(torch.rand(n, device=dev, generator=g) < 0.5) for _ in range(ns)]
    dense, bst = [1048576, 32768, 64, 1], [0, 64, 0, 1]
    reps = max(8, args.ops_launches)     # launches per recorded graph, rotating over the buffer sets
    results = {}
    side = torch.cuda.Stream()
    marker = torch.zeros(4, dtype=torch.int32, device=dev)
    one = ctypes.c_int32(1)

    def timed(name, fn, nset, bytes_, kernels_per_call=1):
        """A marker launch, >= 10 eager warm-up launches, then `reps` launches recorded into ONE HIP
        graph (back to back, no host in between); the graph is replayed untimed until >= 30 ms of
        continuous work have passed, then timed replays run between one pair of events on the
        launching stream."""
        with torch.cuda.stream(side):
            check(lib().rmlk_hip_write_small(side.cuda_stream, marker.data_ptr(), ctypes.byref(one), 4),
                  "rmlk_hip_write_small")
            for i in range(max(10, nset)):
                fn(i % nset)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for i in range(reps):
                    fn(i % nset)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(side)
            graph.replay()
            e1.record(side)
            side.synchronize()
            first_ms = max(e0.elapsed_time(e1), 1e-3)
            n_warm = 0 if args.ops_quick else min(200, int(30.0 / first_ms) + 1)
            for _ in range(n_warm):
                graph.replay()
            n_timed = 1 if args.ops_quick else max(3, min(50, int(20.0 / first_ms)))
            e0.record(side)
            for _ in range(n_timed):
                graph.replay()
            e1.record(side)
            side.synchronize()
        us = e0.elapsed_time(e1) / (n_timed * reps) * 1e3
        results[name] = {"us_per_call_with_launch_gaps": round(us, 2), "algorithmic_bytes": bytes_,
                         "calls_timed": n_timed * reps, "kernels_per_call": kernels_per_call,
                         "buffer_sets": nset, "launches_per_graph": reps}
        log(f"[ops] {name}: {us:.2f} us/call with launch gaps, {bytes_ / us / 1e6:.2f} TB/s")
        del graph

    # (before the first marker launch, so that a kernel trace split at the markers does not see them)
    half = n * 2
    sink = torch.zeros(4096, dtype=torch.int32, device=dev)
    big = [torch.empty(CALIBRATION_COPY_BYTES // 4, device=dev) for _ in range(4)]
    for t in big:
        t.normal_(generator=g)
    clock = {}
    # read-only launches of the sizes a decode step's one-row products stream (o 16 MiB, q/k/v 24,
    # down 64, gate/up 128), rotating through 1 GiB: what a chain of such launches costs at the least
    for mib in (16, 24, 64, 128):
        nbytes = mib << 20
        per_buf = CALIBRATION_COPY_BYTES // nbytes
        pieces = [b_[j * (nbytes // 4):(j + 1) * (nbytes // 4)] for b_ in big for j in range(per_buf)]
        blocks = nbytes // 32768
        n_l = 48
        stamps = torch.zeros(n_l, blocks, 2, dtype=torch.int64, device=dev)
        with torch.cuda.stream(side):
            fn = lambda i: k.stream_yardstick(k.YARDSTICK_READ, pieces[i % len(pieces)], sink, nbytes,  # noqa: E731
                                              stamps=stamps[i % n_l], stream=side.cuda_stream)
            for i in range(len(pieces)):
                fn(i)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for i in range(n_l):
                    fn(i)
            for _ in range(10 if args.ops_quick else 60):
                graph.replay()
            side.synchronize()
        st = stamps.cpu().numpy().astype(np.int64)
        first, last_end = st[:, :, 0].min(1), st[:, :, 1].max(1)
        clock[f"read_{mib}MiB"] = {"launches": n_l,
                                   "first_start_to_last_end_us": round(float(((last_end - first) * 0.01).mean()), 2),
                                   "start_to_start_us": round(float(np.median((first[1:] - first[:-1]) * 0.01)), 2)}
        log(f"[ops] in-kernel clock, read {mib} MiB: {clock[f'read_{mib}MiB']}")
        del graph, stamps
    for name, kind, nbytes, blocks in (("read_33MB", k.YARDSTICK_READ, n * 4, n * 4 // 32768),
                                       ("copy_17MB_17MB", k.YARDSTICK_COPY, half, half // 16384),
                                       ("copy_33MB_33MB", k.YARDSTICK_COPY, n * 4, n * 4 // 16384)):
        stamps = torch.zeros(reps, blocks, 2, dtype=torch.int64, device=dev)
        with torch.cuda.stream(side):
            fn = lambda i: k.stream_yardstick(kind, xs[i % ns], sink if kind == k.YARDSTICK_READ else ys[i % ns],  # noqa: E731
                                              nbytes, stamps=stamps[i % reps], stream=side.cuda_stream)
            for i in range(ns):
                fn(i)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for i in range(reps):
                    fn(i)
            for _ in range(20 if args.ops_quick else 200):
                graph.replay()
            side.synchronize()
        st = stamps.cpu().numpy().astype(np.int64)          # 100 MHz: 10 ns per tick
        first, last_start, last_end = st[:, :, 0].min(1), st[:, :, 0].max(1), st[:, :, 1].max(1)
        span = (last_end - first) * 0.01
        gap = (first[1:] - last_end[:-1]) * 0.01
        clock[name] = {"launches": int(reps), "first_start_to_last_end_us": round(float(span.mean()), 2),
                       "min": round(float(span.min()), 2), "max": round(float(span.max()), 2),
                       "first_start_to_last_start_us": round(float(((last_start - first) * 0.01).mean()), 2),
                       "last_end_to_next_first_start_us": round(float(gap.mean()), 2),
                       "start_to_start_us": round(float(((first[1:] - first[:-1]) * 0.01).mean()), 2),
                       "by_buffer_set_us": [round(float(span[np.arange(reps) % ns == j].mean()), 2) for j in range(ns)]}
        log(f"[ops] in-kernel clock, {name}: {clock[name]}")
        del graph, stamps
    # What a SIMD does with other instructions beside fp32 MFMAs (one block per compute unit, two
    # wavefronts per SIMD): cycles per MFMA of a chain with 0..16 independent v_fma_f32 behind each,
    # what a second wavefront's chain of dependent v_fma_f32 gets done meanwhile, and cycles per
    # MFMA of independent MFMAs with an instruction behind every fourth.
    issue = {}
    iters = 2000
    cyc = torch.zeros(256, 8, dtype=torch.int64, device=dev)
    for nv in (0, 4, 8, 12, 16):
        for second in (False, True):
            cyc.zero_()
            k.issue_yardstick(nv, second, iters, cyc)
            torch.cuda.synchronize()
            c = cyc.cpu().numpy().astype(np.float64)
            row = {"cycles_per_mfma": round(float(c[:, :4].mean() / (16 * iters)), 1)}
            if second:
                row["second_wavefront_cycles_per_64_fma"] = round(float(c[:, 4:].mean() / iters), 1)
            issue[f"{nv}_fma_per_mfma" + ("_with_second_wavefront" if second else "")] = row
    for kind, what in ((100, "nothing"), (101, "v_add_u32"), (102, "ds_read_b128"),
                       (103, "v_add_u32_then_the_ds_read_b128_that_waits_for_it")):
        cyc.zero_()
        k.issue_yardstick(kind, False, iters, cyc)
        torch.cuda.synchronize()
        c = cyc.cpu().numpy().astype(np.float64)
        per = float(c[:, :4].mean() / (16 * iters))
        issue[f"independent_mfmas_{what}_behind_every_4th"] = {"cycles_per_mfma": round(per, 2),
                                                              "cycles_per_occurrence": round((per - 64.0) * 4, 1)}
    cyc.zero_()
    log(f"[ops] issue yardstick: {issue}")
    clock["issue"] = issue
    # ---- yardsticks: an almost empty launch and a plain 256 MiB copy -------------------------------
    timed("launch_floor", lambda i: check(lib().rmlk_hip_fill(side.cuda_stream, k.INT32, 1, ctypes.byref(one),
                                                              marker.data_ptr()), "rmlk_hip_fill"), 1, 4)
    timed("copy_256MiB", lambda i: check(lib().rmlk_hip_memcpy_dtod(
        side.cuda_stream, big[2 + i % 2].data_ptr(), big[i % 2].data_ptr(), CALIBRATION_COPY_BYTES),
        "rmlk_hip_memcpy_dtod"), 2, 2 * CALIBRATION_COPY_BYTES)
    del big
    # minimal streaming kernels over the same rotating buffers as the operators below: what this chip
    # does with 33.5 MB read, 16.8 + 16.8 MB copied and 33.5 + 33.5 MB copied when a kernel does
    # nothing else. yardstick_clock adds, from clocks read inside those kernels, how a launch's time
    # splits into the memory system's part and what lies between two launches.
    timed("yardstick_read_33MB", lambda i: k.stream_yardstick(k.YARDSTICK_READ, xs[i], sink, n * 4,
                                                              stream=side.cuda_stream), ns, n * 4)
    timed("yardstick_copy_17MB_17MB", lambda i: k.stream_yardstick(k.YARDSTICK_COPY, xs[i], ys[i], half,
                                                                   stream=side.cuda_stream), ns, 2 * half)
    timed("yardstick_copy_33MB_33MB", lambda i: k.stream_yardstick(k.YARDSTICK_COPY, xs[i], ys[i], n * 4,
                                                                   stream=side.cuda_stream), ns, 2 * n * 4)
    # ---- configs[1] ---------------------------------------------------------------------------------
    timed("add", lambda i: k.binary(k.ADD, xs[i], bs[i], ys[i], shp, dense, bst), ns, 2 * n * 4 + 8192)
    timed("mul", lambda i: k.binary(k.MUL, xs[i], bs[i], ys[i], shp, dense, bst), ns, 2 * n * 4 + 8192)
    timed("div", lambda i: k.binary(k.DIV, xs[i], bs[i], ys[i], shp, dense, bst), ns, 2 * n * 4 + 8192)
    timed("where", lambda i: k.where(xs[i], bs[i], conds[i], ys[i], shp, dense, bst, dense), ns,
          2 * n * 4 + n + 8192)
    rm_out = torch.empty(4096, device=dev)
    timed("reduce_mean", lambda i: k.reduce_mean(xs[i], rm_out, [4096, 2048], [1]), ns, n * 4 + 16384)
    timed("transpose", lambda i: k.transpose(xs[i], ys[i], [1, 2048, 32, 64], [0, 2, 1, 3]), ns,
          2 * 2048 * 32 * 64 * 4)
    table = torch.randn(128256, 2048, device=dev, generator=g)
    idx = [torch.randint(0, 128256, (2048,), device=dev, generator=g) for _ in range(ns)]
    timed("gather", lambda i: k.gather(table, idx[i], ys[i], [128256, 2048], 0), ns,
          2 * 2048 * 2048 * 4 + 2048 * 8)
    del table
    sx = [torch.randn(32 * 2048, 2048, device=dev, generator=g) for _ in range(2)]
    mask = torch.triu(torch.full((2048, 2048), float("-inf"), device=dev), 1)
    for t in sx:
        t.view(32, 2048, 2048).add_(mask)
    so = [torch.empty_like(sx[0]) for _ in range(2)]
    timed("softmax", lambda i: k.softmax(sx[i], so[i], 65536, 2048, 1), 2, 2 * sx[0].numel() * 4)
    # ---- fused chains at the shapes they take in the Llama prefill (S = 2048) ---------------------
    gam = torch.rand(2048, device=dev, generator=g) + 0.5
    timed("fused_rmsnorm", lambda i: k.rmsnorm(xs[i], gam, ys[i], 4096, 2048, 1e-5), ns,
          2 * n * 4 + 8192)
    timed("fused_rmsnorm_recip", lambda i: k.rmsnorm(xs[i], gam, ys[i], 4096, 2048, 1e-5, True), ns,
          2 * n * 4 + 8192)
    sums = [torch.empty(n, device=dev) for _ in range(ns)]
    timed("fused_add_rmsnorm", lambda i: k.add_rmsnorm(xs[i], xs[(i + 1) % ns], gam, sums[i], ys[i],
                                                       4096, 2048, 1e-5), ns, 4 * n * 4 + 8192)
    del sums
    timed("fused_swiglu", lambda i: k.swiglu(xs[i], xs[(i + 1) % ns], ys[i]), ns, 3 * n * 4)
    cs_tab = torch.randn(2 * 2048 * 64, device=dev, generator=g)
    rot_shape = [1, 64, 2048, 64]       # the [1, 2048, 64, 64] projection read head-major
    timed("fused_rotary", lambda i: k.rotary(xs[i], cs_tab[:2048 * 64], cs_tab[2048 * 64:], ys[i], rot_shape,
                                             [0, 64, 64 * 64, 1], [0, 0, 64, 1], [0, 0, 64, 1]), ns,
          2 * n * 4 + 2 * 2048 * 64 * 4)
    msk = torch.triu(torch.full((2048, 2048), float("-inf"), device=dev), 1)
    plain = [torch.randn(32 * 2048, 2048, device=dev, generator=g) for _ in range(2)]
    timed("fused_scale_mask_softmax",
          lambda i: k.scale_mask_softmax(plain[i], msk, so[i], [1, 32, 2048, 2048], [0, 0, 2048, 1], 8.0),
          2, 2 * plain[0].numel() * 4 + 2048 * 2048 * 4)
    del plain
    # ---- configs[4] shapes: KV-cache / indexing stress ---------------------------------------------
    kv_n = 8 * 8192 * 64
    nk = ns * 2
    caches = [torch.randn(kv_n, device=dev, generator=g) for _ in range(nk)]
    outs = [torch.empty(kv_n, device=dev) for _ in range(nk)]
    rows = [torch.randn(8 * 64, device=dev, generator=g) for _ in range(ns)]
    sidx = [torch.tensor([[0, h, int(p)] for h in range(8)], device=dev, dtype=torch.int64)
            for p in np.random.default_rng(5).integers(0, 8192, size=ns)]

    timed("scatter_nd_copy", lambda i: k.scatter_nd_copy(sidx[i % ns], rows[i % ns], caches[i % nk], outs[i % nk],
                                                         [1, 8, 8192, 64], 8, 3), nk,
          2 * kv_n * 4 + 8 * 64 * 4 + 192)
    timed("scatter_nd_inplace", lambda i: k.scatter_nd(sidx[i % ns], rows[i % ns], caches[i % nk],
                                                       [1, 8, 8192, 64], 8, 3), nk, 8 * 64 * 4 + 192)
    timed("slice_kv", lambda i: k.slice_(caches[i % nk], outs[i % nk], [1, 8, 8192, 64], [0, 0, 0, 0],
                                         [1, 1, 1, 1], [1, 8, 8191, 64]), nk, 2 * 8 * 8191 * 64 * 4)

    timed("concat_kv", lambda i: k.concat([caches[i % nk][:8 * 8191 * 64], rows[i % ns]], outs[i % nk],
                                          [[1, 8, 8191, 64], [1, 8, 1, 64]], [1, 8, 8192, 64], 2), nk,
          2 * kv_n * 4)
    del caches, outs
    table = torch.randn(128256, 2048, device=dev, generator=g)
    idx4 = [torch.randint(0, 128256, (4096,), device=dev, generator=g) for _ in range(ns)]
    g4 = [torch.empty(4096 * 2048, device=dev) for _ in range(ns)]
    timed("gather_4096", lambda i: k.gather(table, idx4[i], g4[i], [128256, 2048], 0), ns,
          2 * 4096 * 2048 * 4 + 4096 * 8)
    del table, g4
    tri_in = [t.view(-1)[:8192 * 8192] for t in sx]
    tri_out = [t.view(-1)[:8192 * 8192] for t in so]
    timed("trilu_8192", lambda i: k.trilu(tri_in[i], tri_out[i], 1, 8192, 8192, True, 1), 2,
          2 * 8192 * 8192 * 4)
    eq_out = torch.empty(8192 * 8192, dtype=torch.bool, device=dev)
    full = [8192, 8192]
    dn = [8192, 1]
    timed("equal_f32_8192", lambda i: k.binary(k.EQUAL, tri_in[i], tri_in[1 - i], eq_out, full, dn, dn),
          2, 2 * 8192 * 8192 * 4 + 8192 * 8192)
    timed("greater_f32_8192", lambda i: k.binary(k.GREATER, tri_in[i], tri_in[1 - i], eq_out, full, dn, dn),
          2, 2 * 8192 * 8192 * 4 + 8192 * 8192)
    i64a = [torch.randint(0, 100, (8192 * 8192,), device=dev, generator=g) for _ in range(2)]
    timed("equal_i64_8192", lambda i: k.binary(k.EQUAL, i64a[i], i64a[1 - i], eq_out, full, dn, dn), 2,
          2 * 8192 * 8192 * 8 + 8192 * 8192)
    with torch.cuda.stream(side):          # closing marker: the last op's segment ends here
        check(lib().rmlk_hip_write_small(side.cuda_stream, marker.data_ptr(), ctypes.byref(one), 4),
              "rmlk_hip_write_small")
        side.synchronize()
    print(json.dumps({"suite": "ops", "note": "us_per_call_with_launch_gaps: HIP events around replays of a "
                      "recorded graph of rotating launches; kernel durations come from rocprofv3 "
                      "--kernel-trace of this command (bench.py --summarize-ops)",
                      "yardstick_clock": {"note": "the yardstick launches once more, 100 per recorded graph over the "
                                          "rotating buffers, each block noting the 100 MHz clock at its start "
                                          "and end: times of the last replay, per launch", **clock},
                      "results": results}))


OPS_MARKER_KERNEL = "write_small_kernel"


def _ops_segments(csv_path):
    """Dispatch rows of a rocprofv3 CSV (kernel trace or counter collection) of `--suite ops`, in
    start order, cut at the marker launches: one list of this library's dispatches per op."""
    import csv
    rows = list(csv.DictReader(open(csv_path)))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    segments, cur = [], None
    for r in rows:
        name = r["Kernel_Name"]
        if OPS_MARKER_KERNEL in name:
            if cur is not None:
                segments.append(cur)
            cur = []
        elif cur is not None and "rmlk::" in name:
            cur.append(r)
    return segments


def _short_kernel_name(name):
    import re
    name = re.sub(r"rmlk::\(anonymous namespace\)::", "", name)
    name = re.sub(r"^void ", "", name).replace("rmlk::", "")
    cut = name.find("(")
    return (name if cut < 0 else name[:cut])[:64]


def summarize_ops(args):
    """Markdown table per op of `--suite ops` from its JSON line and the rocprofv3 CSVs of the same
    command: kernel-trace durations of the timed launches (the last calls_timed of each op), and,
    when given, FETCH_SIZE / WRITE_SIZE per call scaled by what the counters read for the 256 MiB
    copy of the same run."""
    res = json.loads([l for l in open(args.summarize_ops) if l.startswith("{")][-1])["results"]
    names = list(res)
    segs = _ops_segments(args.kernel_trace)
    assert len(segs) == len(names), (len(segs), len(names))
    pmc = {}
    for label, path in (("FETCH_SIZE", args.pmc_fetch), ("WRITE_SIZE", args.pmc_write)):
        if not path:
            continue
        psegs = _ops_segments(path)
        assert len(psegs) == len(names), (label, len(psegs), len(names))
        per_call = {}
        for nm, seg in zip(names, psegs):
            vals = [float(r["Counter_Value"]) for r in seg if r["Counter_Name"] == label]
            kpc = res[nm]["kernels_per_call"]
            per_call[nm] = sum(vals) / (len(vals) / kpc) if vals else None
        unit = (CALIBRATION_COPY_BYTES / 1024.0) / per_call["copy_256MiB"]
        pmc[label] = ({nm: None if v is None else v * unit * 1024.0 for nm, v in per_call.items()}, unit)
    floor = None
    print("| op | kernel(s) | grid x block | timed launches | avg us | min us | algorithmic MB | TB/s | % of 8 TB/s"
          + (" | fetched MB | written MB | moved / algorithmic" if pmc else "") + " |")
    print("|---|---|---|---|---|---|---|---|---|" + ("---|---|---|" if pmc else ""))
    for nm, seg in zip(names, segs):
        r = res[nm]
        kpc = r["kernels_per_call"]
        timed_rows = seg[-r["calls_timed"] * kpc:]
        durs = [int(x["End_Timestamp"]) - int(x["Start_Timestamp"]) for x in timed_rows]
        calls = [sum(durs[i:i + kpc]) / 1e3 for i in range(0, len(durs), kpc)]
        avg, mn = sum(calls) / len(calls), min(calls)
        kernels = []
        for x in timed_rows[:kpc]:
            kn = _short_kernel_name(x["Kernel_Name"])
            wg = int(x["Workgroup_Size_X"]) if "Workgroup_Size_X" in x else int(x["Workgroup_Size"])
            gs = int(x["Grid_Size_X"]) if "Grid_Size_X" in x else int(x["Grid_Size"])
            kernels.append((kn, f"{gs // wg} x {wg}"))
        mb = r["algorithmic_bytes"] / 1e6
        if nm == "launch_floor":
            floor = avg
        line = (f"| {nm} | {' + '.join(kk for kk, _ in kernels)} | {' + '.join(gg for _, gg in kernels)} | "
                f"{len(calls)} | {avg:.2f} | {mn:.2f} | {mb:.1f} | {mb / avg:.2f} | {mb / avg / 8.0 * 100:.0f}")
        if pmc:
            f = pmc.get("FETCH_SIZE", ({}, 0))[0].get(nm)
            w = pmc.get("WRITE_SIZE", ({}, 0))[0].get(nm)
            moved = (f or 0) + (w or 0)
            line += (f" | {'-' if f is None else f'{f / 1e6:.1f}'} | {'-' if w is None else f'{w / 1e6:.1f}'}"
                     f" | {moved / r['algorithmic_bytes']:.2f}" if r["algorithmic_bytes"] > 4096 else " | - | - | -")
        print(line + " |")
    for label, (_, unit) in pmc.items():
        print(f"\n{label}: one counter unit = {unit:.3f} KiB (from the 256 MiB copy of the same run).")
    # which launches are the fast ones: by place in the recorded graph and by buffer set
    import numpy as np
    print("\n| op | p10 us | p50 us | p90 us | first launch of a replay | other launches | launches on buffer set 0 "
          "| on other sets | start-to-start p50 us |")
    print("|---|---|---|---|---|---|---|---|---|")
    for nm, seg in zip(names, segs):
        r = res[nm]
        kpc, nset = r["kernels_per_call"], r["buffer_sets"]
        if kpc != 1 or r["algorithmic_bytes"] <= 4096:
            continue
        rows = seg[-r["calls_timed"]:]
        st = np.array([int(x["Start_Timestamp"]) for x in rows])
        d = np.array([int(x["End_Timestamp"]) for x in rows]) - st
        d = d / 1e3
        per_graph = int(r.get("launches_per_graph", 100))
        pos = np.arange(len(d)) % per_graph
        bset = pos % nset
        p10, p50, p90 = np.percentile(d, [10, 50, 90])
        s2s = np.diff(st) / 1e3
        print(f"| {nm} | {p10:.2f} | {p50:.2f} | {p90:.2f} | {d[pos == 0].mean():.2f} | {d[pos != 0].mean():.2f} | "
              f"{d[bset == 0].mean():.2f} | {d[bset != 0].mean():.2f} | {np.median(s2s):.2f} |")


def run_graph_suite(args):
    """BASELINE configs[0], [2] and [4] as graphs through the session, with pattern fusion and with
    one kernel per node: replays of the recorded HIP graph timed on the device, and one eager pass
    with HIP events per node for the per-operator figures. A torch `bitwise_not` launch marks the
    start of every timed block in a kernel trace (`bench.py --summarize-graph`)."""
    import numpy as np
    import torch
    from rmlk_amd import graphs, runtime
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    marker = torch.zeros(4, dtype=torch.int32, device="cuda:0")
    if args.suite == "c1":
        graph, feeds = graphs.rmsnorm_matmul_graph(seed=1)
        workload = "BASELINE configs[0]: decomposed RMSNorm [1,128,2048] + MatMul [2048,8192], fp32"
    elif args.suite == "c3":
        graph, feeds = graphs.decoder_layer_graph(seed=3, seq=2048, bf16_values=args.bf16_values)
        workload = "BASELINE configs[2]: one Llama-3.2-1B-shaped decoder layer, prefill S=2048, fp32"
        if args.bf16_values:
            workload += ("; weights that are bfloat16 values held as floats (16-bit storage where lossless)" +
                         (", many-row products of the fused session as bfloat16 pieces on the bf16 matrix cores"
                          if args.bf16_pieces else ""))
    else:
        graph, feeds = graphs.kv_stress_graph(seed=5)
        workload = "BASELINE configs[4]: indexing / KV-cache stress graph at length 8192"
    mm_ops = ("MatMul", "rmlk.MatMulGroup", "rmlk.MatMulGroupSwiGLU", "rmlk.MatMulAddRMSNorm",
              "rmlk.MatMulConst", "rmlk.AttnMatMul")
    blocks, out = [], {"suite": args.suite, "workload": workload, "modes": {}}
    reference = None
    for mode, fuse in (("fused", True), ("one_kernel_per_node", False)):
        inst = runtime.Builder.from_graph(graph).build(0, fuse=fuse, bf16_pieces=fuse and args.bf16_pieces)
        got = inst.run(feeds)                      # first run fills the pool; outputs kept for the check
        if reference is None:
            reference = got
        else:
            for name in reference:
                a, b = reference[name], got[name]
                if a.dtype.kind == "f":
                    np.testing.assert_allclose(a, b, rtol=2e-3, atol=2e-4, err_msg=name)
                else:
                    assert np.array_equal(a, b), name
        for name, arr in feeds.items():
            inst.set_input(name, arr)
        inst.capture()
        for _ in range(max(args.warmup, 3)):
            inst.replay()
        inst.sync()
        marker.bitwise_not_()              # the mark in a kernel trace (the session never launches this)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            inst.replay_enqueue()
        inst.check()
        ms = (time.perf_counter() - t0) / args.steps * 1e3
        marker.bitwise_not_()              # end of the timed block; what follows up to the next mark is not timed
        torch.cuda.synchronize()
        blocks.append({"label": mode, "replays": args.steps})
        blocks.append(None)
        # per-node events on one eager pass (they add a cache write-back after every node)
        for name, arr in feeds.items():
            inst.set_input(name, arr)
        inst.set_profiling(True)
        inst.execute()
        inst.set_profiling(False)
        per_op, mm_us, mm_flops = {}, 0.0, 0.0
        for st in inst.node_stats():
            if st["micros"] <= 0:
                continue
            d = per_op.setdefault(st["op"], {"n": 0, "us": 0.0, "bytes": 0.0})
            d["n"] += 1
            d["us"] += st["micros"]
            d["bytes"] += st["bytes"]
            if st["op"] in mm_ops:
                mm_us += st["micros"]
                mm_flops += st["flops"]
        out["modes"][mode] = {
            "ms_per_pass_device_replay": round(ms, 4), "nodes": len(graph.nodes),
            "fused_nodes": inst.fused_nodes,
            "matmul_us_with_events": round(mm_us, 1),
            "matmul_tflops_with_events": round(mm_flops / mm_us / 1e6, 2) if mm_us else None,
            "ops_with_events": {op: {"n": d["n"], "us": round(d["us"], 1),
                                     "gbs": round(d["bytes"] / d["us"] / 1e3, 1)}
                                for op, d in sorted(per_op.items(), key=lambda kv: -kv[1]["us"])}}
        log(f"[{args.suite}] {mode}: {ms:.3f} ms per pass (device replay), MatMul nodes {mm_us:.1f} us with events")
        inst.close()
    out["trace_blocks"] = blocks[:-1]
    print(json.dumps(out))


GRAPH_MARKER_KERNEL = "bitwise_not"


def summarize_graph(args):
    """Kernels of every timed block of a graph suite (split at the marker launches), grouped by
    kernel and grid: launches per replay, average and summed duration per replay."""
    import csv
    import statistics
    res = json.loads([l for l in open(args.summarize_graph) if l.startswith("{")][-1])
    rows = list(csv.DictReader(open(args.kernel_trace)))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    segments, cur = [], None
    for r in rows:
        if GRAPH_MARKER_KERNEL in r["Kernel_Name"]:
            if cur is not None:
                segments.append(cur)
            cur = []
        elif cur is not None and "rmlk::" in r["Kernel_Name"]:
            cur.append(r)
    blocks = res["trace_blocks"]
    assert len(segments) == len(blocks), (len(segments), len(blocks))
    print(f"Workload: {res['workload']}\n")
    for blk, seg in zip(blocks, segments):
        if blk is None:
            continue
        reps = blk["replays"]
        n_launch = len(seg)
        per_replay = n_launch // reps if n_launch % reps == 0 else None
        timed = seg[:per_replay * reps] if per_replay else seg
        groups = {}
        for x in timed:
            key = (_short_kernel_name(x["Kernel_Name"]),
                   f"{int(x['Grid_Size_X']) // int(x['Workgroup_Size_X'])}x{int(x['Grid_Size_Y'])}x{int(x['Grid_Size_Z'])}")
            groups.setdefault(key, []).append((int(x["End_Timestamp"]) - int(x["Start_Timestamp"])) / 1e3)
        total = sum(sum(v) for v in groups.values()) / reps
        mode = res["modes"][blk["label"]]
        print(f"### {blk['label']}: {n_launch // reps} launches per pass, {total:.1f} us of kernel time per pass, "
              f"{mode['ms_per_pass_device_replay'] * 1e3:.1f} us per replay on the host clock\n")
        print("| kernel | blocks | launches per pass | avg us | min us | us per pass |")
        print("|---|---|---|---|---|---|")
        for (name, grid), v in sorted(groups.items(), key=lambda kv: -sum(kv[1])):
            print(f"| {name} | {grid} | {len(v) / reps:g} | {statistics.mean(v):.2f} | {min(v):.2f} | {sum(v) / reps:.1f} |")
        print()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--decode", type=int, default=128)
    ap.add_argument("--cpu-tokens", type=int, default=512)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--weights", default="f32", choices=["f32", "auto", "f16", "bf16"],
                    help="llama suite: how the session stores the constant MatMul weights (arithmetic is "
                         "fp32 in every case). The reference and the headline figure are f32; auto: 16-bit "
                         "where every float of a matrix is a bfloat16 / half value already (nothing lost); "
                         "f16 / bf16: rounded to that type (the oracle leg is skipped: it walks the "
                         "unrounded graph)")
    ap.add_argument("--no-variants", action="store_true",
                    help="llama suite: skip the run over bfloat16-valued weights that the default run adds")
    ap.add_argument("--bf16-values", action="store_true",
                    help="llama suite: synthetic weights that are bfloat16 values held as floats, as a "
                         "checkpoint trained in bfloat16 and exported as float has them")
    ap.add_argument("--bf16-pieces", action="store_true",
                    help="llama suite: many-row products over weights held as bfloat16 values split their "
                         "fp32 operand into three bfloat16 pieces (exactly) and run on the bf16 matrix cores "
                         "(fp32 results; needs --bf16-values with --weights auto, or --weights bf16)")
    ap.add_argument("--tiny", action="store_true", help="2-layer toy shape (plumbing check only)")
    ap.add_argument("--suite", default="llama", choices=["llama", "ops", "c1", "c3", "c5"])
    ap.add_argument("--ops-launches", type=int, default=100, help="ops suite: launches per recorded graph")
    ap.add_argument("--ops-quick", action="store_true",
                    help="ops suite: one replay per op, no settling (for counter runs, which serialise launches)")
    ap.add_argument("--summarize-ops", metavar="JSON", help="print the per-op table from an ops-suite JSON "
                    "line and the rocprofv3 CSVs of the same command (no GPU needed)")
    ap.add_argument("--summarize-graph", metavar="JSON", help="print the per-kernel table of a c1/c3/c5 "
                    "suite from its JSON line and the rocprofv3 kernel trace of the same command")
    ap.add_argument("--kernel-trace", metavar="CSV")
    ap.add_argument("--pmc-fetch", metavar="CSV")
    ap.add_argument("--pmc-write", metavar="CSV")
    args = ap.parse_args()
    if args.summarize_ops:
        summarize_ops(args)
        return
    if args.summarize_graph:
        summarize_graph(args)
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one MI355X: the operator path has no multi-GPU part "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if args.suite == "ops":
        run_ops_suite(args)
        return
    if args.suite in ("c1", "c3", "c5"):
        run_graph_suite(args)
        return
    result = run_llama(args)
    if args.weights == "f32" and not args.bf16_values and not args.tiny and not args.no_variants:
        # The same graph with weights that are bfloat16 values held as floats - what a released
        # Llama-3.2 checkpoint exported as fp32 looks like - under default session flags: the session
        # holds them in 16 bits by itself (nothing is lost). Reported beside the headline, never as it.
        import copy
        v = copy.copy(args)
        v.bf16_values, v.weights, v.no_cpu, v.steps, v.warmup = True, "auto", True, 3, 1
        r = run_llama(v)
        result["variant_bf16_valued_weights"] = {
            "what": "same graph, weights rounded to bfloat16 values and held as fp32 initializers; default "
                    "session flags (16-bit storage where lossless), fp32 arithmetic",
            "weight_storage": r["weight_storage"], "prefill_tok_s": r["value"],
            "decode_ms_per_token": r["decode_ms_per_token"],
            "decode_device_ms_per_token": r["decode_device_ms_per_token"],
            "decode_weight_gbs": r["decode_weight_gbs"],
            "session_device_bytes_after_build": r["memory"]["session_device_bytes_after_build"]}
        # ... and with the prefill's products on the bf16 matrix cores: the fp32 operand as three
        # bfloat16 pieces whose sum it is exactly, exact products, fp32 accumulation
        v.bf16_pieces = True
        r = run_llama(v)
        result["variant_bf16_valued_weights"]["prefill_tok_s_products_as_bf16_pieces"] = r["value"]
        result["variant_bf16_valued_weights"]["prefill_ms_products_as_bf16_pieces"] = r["ms_per_step"]
        result["variant_bf16_valued_weights"]["prefill_products_on_bf16_matrix_cores"] = \
            r["prefill_products_on_bf16_matrix_cores"]
        result["variant_bf16_valued_weights"]["roofline_products_as_bf16_pieces"] = {
            k_: r["roofline"][k_] for k_ in ("bound", "kernel", "achieved", "peak", "unit", "frac", "avg_launch_us",
                                             "fp32_equivalent_tflops", "note")}
    print(json.dumps(result))


if __name__ == "__main__":
    main()

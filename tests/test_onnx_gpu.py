"""Sessions built from `.onnx` files, on the GPU: graphs serialised by PyTorch's exporter against the
outputs PyTorch computed (tests/golden/torch_*.{onnx,npz}), and this package's benchmark graphs
written to ONNX, read back by the native reader and run against the directly built graph."""
import os

import numpy as np
import pytest

from helpers import assert_close, assert_exact

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("name", ["torch_norm_proj_softmax", "torch_decoder_block"])
@pytest.mark.parametrize("fuse", [True, False])
def test_pytorch_export_matches_pytorch_output(device, name, fuse):
    from rmlk_amd import runtime
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    inst = runtime.Builder.from_onnx_path(os.path.join(GOLDEN, name + ".onnx")).build(fuse=fuse)
    feeds = {k: z[k] for k in inst.graph.inputs}
    out = inst.run(feeds)["y"]
    assert_close(out, z["y"], rtol=1e-4, atol=1e-5)
    assert inst.memory_stats()["device_syncs"] == 0
    if fuse and name == "torch_decoder_block":
        # 2 RMSNorm (reciprocal form), 2 rotary, SwiGLU, scale+mask+softmax, 2 attention products,
        # those three merged into one attention node, the q/k/v and gate/up MatMul groups, one
        # residual Add merged into the second norm and the o projection merged into that, the
        # gate/up group merged with the SwiGLU, the down projection (constant weights), the two
        # rotary nodes merged into one launch of two row streams
        assert inst.fused_nodes == 16
    inst.close()


def test_dynamic_sequence_of_a_pytorch_export(device):
    """The exported graph has a symbolic sequence dim: other lengths than the traced one run."""
    from oracle import graph as og
    from oracle import onnx_read
    from rmlk_amd import runtime
    path = os.path.join(GOLDEN, "torch_norm_proj_softmax.onnx")
    inst = runtime.Builder.from_onnx_path(path).build()
    lg = onnx_read.read_onnx(path)
    for seq in (1, 9):
        x = np.random.default_rng(seq).standard_normal((2, seq, 64), dtype=np.float32)
        assert_close(inst.run({"x": x})["y"], og.run_graph(lg, {"x": x})["y"], rtol=1e-4, atol=1e-5)
    inst.close()


def test_written_llama_graph_runs_like_the_built_one(device, tmp_path):
    from rmlk_amd import graphs, onnx_io, runtime
    cfg = graphs.LlamaConfig.tiny()
    graph = graphs.llama_graph(cfg, seed=4, style="concat")
    path = str(tmp_path / "llama_tiny.onnx")
    onnx_io.save_onnx(graph, path, external_data=True, external_threshold=512)
    feeds = graphs.llama_concat_inputs(cfg, np.random.default_rng(2).integers(0, cfg.vocab, 7), None, 0)
    a = runtime.Builder.from_graph(graph).build()
    b = runtime.Builder.from_onnx_path(path).build()
    assert a.fused_nodes == b.fused_nodes > 0
    ra, rb = a.run(feeds), b.run(feeds)
    assert ra.keys() == rb.keys()
    for k in ra:
        assert_exact(ra[k], rb[k])
    a.close()
    b.close()


def test_written_kv_stress_graph_is_bit_exact(device):
    from rmlk_amd import graphs, onnx_io, runtime
    graph, feeds = graphs.kv_stress_graph(seed=5, heads=2, length=64, head_dim=16, vocab=300,
                                          hidden=32, n_gather=33, mask_n=40)
    a = runtime.Builder.from_graph(graph).build().run(feeds)
    b = runtime.Builder.from_onnx_bytes(onnx_io.graph_to_onnx_bytes(graph)).build().run(feeds)
    for k in a:
        assert_exact(a[k], b[k])

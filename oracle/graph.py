"""CPU oracle for whole graphs (TEST INFRASTRUCTURE ONLY): walks a graph description node by node,
in stored order, exactly like the reference's executor (runtime/src/core/instance.rs:100-112), and
applies oracle.ops to numpy arrays.

A "graph" here is any object with `.nodes` (each with .op, .inputs, .outputs, .attrs),
`.initializers` (name -> ndarray) and `.outputs` (names), which is what rmlk_amd.runtime.Graph keeps
next to its native handle.

Pinning: the single multi-op vector the reference holds (runtime/tests/fixtures/attention_*.f32,
produced by ONNX Runtime CPU, graph in runtime/tests/graphs/attention.rs:15-41) is checked in
tests/test_oracle_golden.py. Whole-graph Llama results have no reference-held vectors and ONNX
Runtime is not installable here: parity unpinned for those beyond per-op pins.
"""
from __future__ import annotations

import numpy as np

from . import ops


def _apply(node, ins, matmul_accumulate):
    op = node.op
    a = node.attrs
    if op == "Add":
        return ops.add(ins[0], ins[1])
    if op == "Sub":
        return ops.sub(ins[0], ins[1])
    if op == "Mul":
        return ops.mul(ins[0], ins[1])
    if op == "Div":
        return ops.div(ins[0], ins[1])
    if op == "Pow":
        return ops.pow_(ins[0], ins[1])
    if op == "Equal":
        return ops.equal(ins[0], ins[1])
    if op == "Greater":
        return ops.greater(ins[0], ins[1])
    if op == "Where":
        return ops.where(ins[0], ins[1], ins[2])
    if op == "Sqrt":
        return ops.sqrt(ins[0])
    if op == "Neg":
        return ops.neg(ins[0])
    if op == "Sin":
        return ops.sin(ins[0])
    if op == "Cos":
        return ops.cos(ins[0])
    if op == "Sigmoid":
        return ops.sigmoid(ins[0])
    if op == "Cast":
        return ops.cast(ins[0], a["to"])
    if op == "ReduceMean":
        axes = None
        if len(ins) > 1 and ins[1] is not None:
            axes = [int(v) for v in np.asarray(ins[1]).reshape(-1)]
        elif "axes" in a:
            axes = list(a["axes"])
        return ops.reduce_mean(ins[0], axes, a.get("keepdims", 1), a.get("noop_with_empty_axes", 0))
    if op == "Softmax":
        return ops.softmax(ins[0], a.get("axis", -1))
    if op == "MatMul":
        return ops.matmul(ins[0], ins[1], accumulate=matmul_accumulate)
    if op == "Transpose":
        return ops.transpose(ins[0], a.get("perm"))
    if op == "Expand":
        return ops.expand(ins[0], np.asarray(ins[1]).reshape(-1))
    if op == "Slice":
        axes = ins[3] if len(ins) > 3 and ins[3] is not None else None
        steps = ins[4] if len(ins) > 4 and ins[4] is not None else None
        return ops.slice_(ins[0], ins[1], ins[2], axes, steps)
    if op == "Concat":
        return ops.concat(ins, a["axis"])
    if op == "Gather":
        return ops.gather(ins[0], ins[1], a.get("axis", 0))
    if op == "ScatterND":
        return ops.scatter_nd(ins[0], ins[1], ins[2], a.get("reduction", "none"))
    if op == "Trilu":
        k = int(np.asarray(ins[1]).reshape(-1)[0]) if len(ins) > 1 and ins[1] is not None else 0
        return ops.trilu(ins[0], k, a.get("upper", 1))
    if op == "Reshape":
        return ops.reshape(ins[0], ins[1], a.get("allowzero", 0))
    if op == "Unsqueeze":
        axes = ins[1] if len(ins) > 1 and ins[1] is not None else a["axes"]
        return ops.unsqueeze(ins[0], axes)
    if op == "Shape":
        return ops.shape_(ins[0], a.get("start", 0), a.get("end"))
    if op == "Range":
        return ops.range_(ins[0], ins[1], ins[2])
    if op == "ConstantOfShape":
        return ops.constant_of_shape(ins[0], a.get("value"))
    if op == "Constant":  # value / value_float(s) / value_int(s), backend/constant.rs
        if "value" in a:
            return np.asarray(a["value"])
        if "value_float" in a:
            return np.array(a["value_float"], dtype=np.float32)
        if "value_floats" in a:
            return np.array(a["value_floats"], dtype=np.float32)
        if "value_int" in a:
            return np.array(a["value_int"], dtype=np.int64)
        return np.array(a["value_ints"], dtype=np.int64)
    raise ops.OracleError(f"unsupported operator {op}")


def run_graph(graph, inputs, matmul_accumulate="f64", keep_all=False):
    """Returns {output name: ndarray} (every value when keep_all)."""
    env = {k: np.asarray(v) for k, v in graph.initializers.items()}
    env.update({k: np.asarray(v) for k, v in inputs.items()})
    for node in graph.nodes:
        ins = [env[n] if n else None for n in node.inputs]
        while ins and ins[-1] is None:
            ins.pop()
        out = _apply(node, ins, matmul_accumulate)
        env[node.outputs[0]] = out
    if keep_all:
        return env
    return {name: env[name] for name in graph.outputs}

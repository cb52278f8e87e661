"""Single-op test helper: the mirror of the reference's `OpTest` (runtime/src/testing.rs:26-194).

Builds a one-op graph through GraphBuilder and runs it through Builder.from_graph(..).build() and
ModelInstance.run, so every case exercises the production dispatch. Feeds are wired to the op in
declaration order; the graph output is always named `y`.
"""
import numpy as np


class OpTest:
    def __init__(self, op: str):
        self.op = op
        self.feeds = []
        self.attrs = []

    def input(self, dims, data, dtype=None):
        arr = np.asarray(data, dtype=dtype).reshape(dims)
        self.feeds.append(("input", f"in{len(self.feeds)}", arr))
        return self

    def constant(self, dims, data, dtype=None):
        arr = np.asarray(data, dtype=dtype).reshape(dims)
        n = sum(1 for f in self.feeds if f[0] == "constant")
        self.feeds.append(("constant", f"const{n}", arr))
        return self

    def attr(self, name, value):
        self.attrs.append((name, value))
        return self

    def output(self, dims):  # shape is inferred by the operator; kept for call-site parity
        return self

    def build(self):
        from rmlk_amd.runtime import GraphBuilder
        g = GraphBuilder()
        names, run_inputs = [], {}
        for kind, name, arr in self.feeds:
            if kind == "input":
                g.input(name, arr.dtype, arr.shape)
                run_inputs[name] = arr
            else:
                g.constant(name, arr)
            names.append(name)
        ob = g.op(self.op, names, ["y"])
        for k, v in self.attrs:
            ob.attr(k, v)
        g.output("y")
        return g.build(), run_inputs

    def run(self):
        from rmlk_amd.runtime import Builder
        graph, run_inputs = self.build()
        inst = Builder.from_graph(graph).build()
        try:
            return inst.run(run_inputs)["y"]
        finally:
            inst.close()

    def run_oracle(self):
        """The same one-op graph on the CPU checker."""
        from oracle.graph import run_graph
        graph, run_inputs = self.build()
        return run_graph(graph, run_inputs)["y"]

    def run_err(self):
        try:
            self.run()
        except Exception as e:  # noqa: BLE001
            return e
        raise AssertionError("expected op to fail, but it succeeded")


def decode(vals, dtype):
    """JSON fixture values -> ndarray ("nan" / "inf" / "-inf" strings are floats)."""
    conv = {"nan": np.nan, "inf": np.inf, "-inf": -np.inf}
    return np.array([conv.get(v, v) if isinstance(v, str) else v for v in vals], dtype=dtype)

#!/usr/bin/env python3
"""Extracts the known-answer vectors the reference's own unit tests hold for the operator path
into tests/golden/reference_cases.json (data only: inputs, attributes, expected outputs).

Run in the build container (the reference tree is not available on the GPU box):

    python tests/golden/extract_reference_cases.py /root/reference

Sources:
  runtime/src/providers/cuda/backend/<op>.rs   #[cfg(test)] OpTest chains (one-op graphs)
  cuda/src/kernels/{reduce_mean,transpose,expand,trilu}.rs  helper-driven kernel tests

The Rust test bodies are read as text and only their literals are evaluated: shapes, data vectors,
attributes and the expected vectors of assert_eq! / assert_close / assert_close_eps. Cases whose
body uses anything else are listed under "skipped" with the reason, so the count is auditable.
"""
from __future__ import annotations

import json
import math
import os
import re
import sys

OPS = ["add", "sub", "mul", "div", "pow", "equal", "greater", "whereop", "sqrt", "neg", "sin", "cos",
       "sigmoid", "cast", "reduce_mean", "softmax", "matmul", "transpose", "expand", "slice",
       "concat", "gather", "scatter_nd", "trilu", "reshape", "unsqueeze", "shape", "range",
       "constant_of_shape", "constant"]

RUST_TYPES = {"f32": "float32", "f64": "float64", "i32": "int32", "i64": "int64", "u8": "uint8",
              "i8": "int8", "u16": "uint16", "i16": "int16", "u32": "uint32", "u64": "uint64",
              "bool": "bool", "f16": "float16", "usize": "int64"}


def split_tests(src: str):
    """Yield (name, body, line) of each #[test] fn in the file's test module."""
    for m in re.finditer(r"#\[test\]\s*(?:#\[[^\]]*\]\s*)*fn\s+(\w+)\s*\(\)\s*\{", src):
        start = m.end()
        depth, i = 1, start
        while depth and i < len(src):
            if src[i] == "{":
                depth += 1
            elif src[i] == "}":
                depth -= 1
            i += 1
        ignored = "#[ignore" in src[m.start():m.end()]
        yield m.group(1), src[start:i - 1], src.count("\n", 0, m.start()) + 1, ignored


def matching(s: str, open_idx: int, open_ch="(", close_ch=")") -> int:
    depth = 0
    for i in range(open_idx, len(s)):
        if s[i] == open_ch:
            depth += 1
        elif s[i] == close_ch:
            depth -= 1
            if depth == 0:
                return i
    raise ValueError("unbalanced")


def split_args(s: str):
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur.strip())
    return out


class Unparsed(Exception):
    pass


SUFFIX = re.compile(r"(?<![A-Za-z_])(-?\d+(?:\.\d*)?(?:[eE][-+]?\d+)?)_?(f32|f64|i32|i64|u8|i8|u16|i16|u32|u64|usize)\b")


def literal_dtype(expr: str):
    m = SUFFIX.search(expr)
    if m:
        return RUST_TYPES[m.group(2)]
    if re.search(r"\b(true|false)\b", expr):
        return "bool"
    if "f16::from_f32" in expr:
        return "float16"
    return None


def eval_vec(expr: str, env: dict):
    """Evaluate a Rust vector / array literal expression to a flat python list."""
    e = expr.strip()
    if e.startswith("&"):
        e = e[1:].strip()
    if e in env:
        return env[e]
    if e.endswith(".clone()") and e[:-8] in env:
        return env[e[:-8]]
    m = re.fullmatch(r"\(\s*(-?\d+)\s*\.\.(=?)\s*(-?\d+)\s*\)\s*\.map\(\|\s*(\w+)\s*\|\s*(.+?)\)\s*\.collect(?:::<[^>]*>)?\(\)", e, re.S)
    if m:
        lo, incl, hi, var, body = int(m.group(1)), m.group(2), int(m.group(3)), m.group(4), m.group(5)
        body = re.sub(r"\bas\s+\w+", "", body)
        body = SUFFIX.sub(r"\1", body)
        rng = range(lo, hi + (1 if incl else 0))
        return [eval(body, {"__builtins__": {}}, {var: v}) for v in rng]
    if re.fullmatch(r"Vec::<\s*\w+\s*>::new\(\)|vec!\s*\[\s*\]|Vec::new\(\)", e):
        return []
    e = re.sub(r"^vec!\s*\[", "[", e)
    e = re.sub(r"(?<=\d)_(?=\d)", "", e)                      # 10_000.0 -> 10000.0
    e = re.sub(r"(-?\d+(?:\.\d*)?)_?f32\.sqrt\(\)", lambda m: repr(float(__import__("numpy").sqrt(__import__("numpy").float32(m.group(1))))), e)
    e = SUFFIX.sub(r"\1", e)
    e = re.sub(r"f16::from_f32\(([^)]*)\)", r"\1", e)
    e = re.sub(r"(?:std::)?f(?:32|64)::consts::PI", repr(math.pi), e)
    e = re.sub(r"(?:std::)?f(?:32|64)::consts::FRAC_PI_2", repr(math.pi / 2), e)
    e = re.sub(r"(?:std::)?f(?:32|64)::consts::FRAC_PI_4", repr(math.pi / 4), e)
    e = re.sub(r"\bf(?:32|64)::NEG_INFINITY\b", "float('-inf')", e)
    e = re.sub(r"\bf(?:32|64)::INFINITY\b", "float('inf')", e)
    e = re.sub(r"\bf(?:32|64)::NAN\b", "float('nan')", e)
    e = re.sub(r"\bi64::MAX\b", str(2 ** 63 - 1), e)
    e = re.sub(r"\bi64::MIN\b", str(-2 ** 63), e)
    e = re.sub(r"\bi32::MAX\b", str(2 ** 31 - 1), e)
    e = re.sub(r"\bi32::MIN\b", str(-2 ** 31), e)
    e = re.sub(r"\btrue\b", "True", e)
    e = re.sub(r"\bfalse\b", "False", e)
    e = re.sub(r"(\d)\.(?=[\s,\]\)])", r"\1.0", e)          # `1.` -> `1.0`
    m = re.fullmatch(r"\[\s*(.+?)\s*;\s*(.+?)\s*\]", e, re.S)  # [x; n]
    if m and "," not in m.group(1):
        count_env = {k: v for k, v in env.items() if isinstance(v, int)}
        return [eval(m.group(1), {"__builtins__": {"float": float}}, {})] * int(
            eval(m.group(2), {"__builtins__": {}}, count_env))
    if not re.fullmatch(r"[\[\]\d\s,.\-+*/eE()TrueFalsfotinan']*", e):
        raise Unparsed(f"expression not literal: {expr.strip()[:60]}")
    v = eval(e, {"__builtins__": {"float": float}}, {})
    if not isinstance(v, (list, tuple)):
        v = [v]
    return list(v)


def jsonable(vals):
    out = []
    for v in vals:
        if isinstance(v, bool):
            out.append(v)
        elif isinstance(v, float):
            out.append("nan" if math.isnan(v) else ("inf" if v == math.inf else
                                                     ("-inf" if v == -math.inf else v)))
        else:
            out.append(v)
    return out


def parse_attr(args):
    name = args[0].strip().strip('"')
    val = args[1].strip()
    m = re.fullmatch(r"AttributeType::(\w+)\((.*)\)", val, re.S)
    if not m:
        raise Unparsed(f"attribute {val[:40]}")
    kind, inner = m.group(1), m.group(2).strip()
    if kind == "Int":
        consts = {"TO_INT32": 6, "TO_INT64": 7, "TO_FLOAT": 1, "TO_DOUBLE": 11, "TO_BOOL": 9,
                  "TO_FLOAT16": 10}
        inner = re.sub(r"\s+as\s+\w+", "", inner)
        if inner in consts:
            return name, consts[inner]
        return name, int(SUFFIX.sub(r"\1", inner))
    if kind == "Float":
        return name, float(SUFFIX.sub(r"\1", inner))
    if kind == "Ints":
        return name, [int(v) for v in eval_vec(inner, {})]
    if kind == "String":
        return name, re.sub(r'\.(to_string|into)\(\)$', "", inner).strip().strip('"')
    raise Unparsed(f"attribute kind {kind}")


def helper_fns(src: str):
    """Zero-argument helper fns of a test module that return a literal vector."""
    out = {}
    for m in re.finditer(r"fn\s+(\w+)\s*\(\)\s*->\s*Vec<\s*(\w+)\s*>\s*\{\s*([^{}]+?)\s*\}", src, re.S):
        try:
            out[m.group(1) + "()"] = eval_vec(m.group(3), {})
            out["__type_" + m.group(1) + "()"] = RUST_TYPES.get(m.group(2))
        except Exception:
            pass
    return out


def parse_optest(body: str, helpers=None):
    env = dict(helpers or {})
    tensors = {}
    for m in re.finditer(r"let\s+(\w+)\s*=\s*Tensor::from_vec\(", body):
        close = matching(body, m.end() - 1)
        a = split_args(body[m.end():close])
        try:
            dims = [int(v) for v in eval_vec(a[0], {})] if a[0].strip() not in ("[]", "&[]") else []
            tensors[m.group(1)] = {"dims": dims, "data": jsonable(eval_vec(a[1], {})),
                                   "dtype": literal_dtype(a[1])}
        except Exception:
            pass
    for m in re.finditer(r"let\s+(?:mut\s+)?(\w+)\s*(?::\s*([^=;]+?))?\s*=\s*([^;]+);", body, re.S):
        name, ty, expr = m.group(1), m.group(2), m.group(3)
        if "OpTest::new" in expr:
            continue
        try:
            if expr.strip() in env:          # let data = zeros();
                env[name] = env[expr.strip()]
                env["__type_" + name] = env.get("__type_" + expr.strip())
                continue
            env[name] = eval_vec(expr, env)
            t = None
            if ty:
                tm = re.search(r"Vec<\s*(\w+)\s*>", ty)
                if tm and tm.group(1) in RUST_TYPES:
                    t = RUST_TYPES[tm.group(1)]
            env["__type_" + name] = t or literal_dtype(expr)
        except Exception:
            pass
    if len(re.findall(r"OpTest::new\(", body)) > 1:
        raise Unparsed("two chained OpTest runs (the second consumes the first's output)")
    m = re.search(r"OpTest::new\(Op::(\w+)\)", body)
    if not m:
        raise Unparsed("no OpTest chain")
    op = m.group(1)
    i = m.end()
    feeds, attrs, out_dims, run_ty, is_err = [], {}, None, None, False
    while True:
        mm = re.match(r"\s*\.\s*(\w+)(?:::<\s*([\w:]+)\s*>)?\s*\(", body[i:])
        if not mm:
            break
        meth, targ = mm.group(1), mm.group(2)
        open_idx = i + mm.end() - 1
        close_idx = matching(body, open_idx)
        args = split_args(body[open_idx + 1:close_idx])
        i = close_idx + 1
        if meth in ("input", "constant"):
            dims = [int(v) for v in eval_vec(args[0], env)] if args[0].strip() not in ("[]", "&[]") else []
            data_expr = args[1]
            data = eval_vec(data_expr, env)
            dt = RUST_TYPES.get(targ) if targ else None
            dt = dt or literal_dtype(data_expr) or env.get("__type_" + data_expr.strip().lstrip("&"))
            feeds.append({"kind": meth, "dims": dims, "data": jsonable(data), "dtype": dt})
        elif meth == "attr":
            tm = re.fullmatch(r"AttributeType::Tensor\(Box::new\((\w+)\)\)", args[1].strip())
            fm = re.fullmatch(r"AttributeType::Floats\((.*)\)", args[1].strip(), re.S)
            if tm and tm.group(1) in tensors:
                attrs[args[0].strip().strip('"')] = {"tensor": tensors[tm.group(1)]}
            elif fm:
                attrs[args[0].strip().strip('"')] = {"floats": jsonable(eval_vec(fm.group(1), {}))}
            else:
                k, v = parse_attr(args)
                attrs[k] = v
        elif meth == "output":
            out_dims = [int(v) for v in eval_vec(args[0], env)] if args[0].strip() not in ("[]", "&[]") else []
        elif meth == "run":
            run_ty = RUST_TYPES.get(targ)
        elif meth == "run_err":
            is_err = True
        elif meth in ("unwrap", "expect"):
            pass
        else:
            raise Unparsed(f"chain method {meth}")
    case = {"op": op, "feeds": feeds, "attrs": attrs, "output_dims": out_dims, "out_dtype": run_ty}
    if is_err or re.search(r"\.unwrap_err\(\)|is_err\(\)", body):
        case["expect_error"] = True
        lit = re.findall(r'contains\("([^"]+)"\)', body)
        case["error_contains"] = lit
        return case
    m = re.search(r"assert_eq!\(\s*out\s*,\s*", body)
    tol = None
    allm = re.search(r"assert!\(out\.iter\(\)\.all\(\|&?x\|\s*\*?x\s*==\s*([-\d.]+)\)\)", body)
    if re.search(r"assert!\(out\.is_empty\(\)\)", body):
        case["expected"], case["tolerance"] = [], 0.0
        return finish_types(case, run_ty)
    if allm and out_dims is not None:
        n = 1
        for d in out_dims:
            n *= d
        case["expected"], case["tolerance"] = [float(allm.group(1))] * n, 0.0
        return finish_types(case, run_ty)
    if m:
        open_idx = body.rfind("(", 0, m.end())
        close_idx = matching(body, open_idx)
        exp_expr = body[m.end():close_idx]
        tol = 0.0
    else:
        m = re.search(r"assert_close(_eps)?\(\s*&out\s*,\s*", body)
        if not m:
            raise Unparsed("no recognised assertion on `out`")
        open_idx = body.rfind("(", 0, m.end())
        close_idx = matching(body, open_idx)
        rest = split_args(body[m.end():close_idx])
        exp_expr = rest[0]
        tol = float(SUFFIX.sub(r"\1", rest[1])) if m.group(1) else 1.2e-7
    case["expected"] = jsonable(eval_vec(exp_expr, env))
    case["tolerance"] = tol
    return finish_types(case, run_ty)


def finish_types(case, run_ty):
    # inputs without a literal suffix take the run type when the op keeps its element type
    for f in case["feeds"]:
        if f["dtype"] is None:
            if all(isinstance(v, bool) for v in f["data"]) and f["data"]:
                f["dtype"] = "bool"
            elif any(isinstance(v, float) or isinstance(v, str) for v in f["data"]):
                f["dtype"] = run_ty if run_ty in ("float32", "float64") else "float32"
            else:
                f["dtype"] = None
    return case


def extract_provider(ref_root: str):
    cases, skipped = [], []
    base = os.path.join(ref_root, "runtime/src/providers/cuda/backend")
    for op in OPS:
        path = os.path.join(base, op + ".rs")
        if not os.path.exists(path):
            continue
        src = open(path).read()
        helpers = helper_fns(src)
        for name, body, line, ignored in split_tests(src):
            cite = f"runtime/src/providers/cuda/backend/{op}.rs:{line}"
            if "OpTest::new" not in body:
                skipped.append({"ref": cite, "test": name, "reason": "host-only helper test"})
                continue
            try:
                case = parse_optest(body, helpers)
                if any(f["dtype"] is None for f in case["feeds"]):
                    raise Unparsed("input element type not stated by a literal suffix")
                case.update({"ref": cite, "test": name, "ignored_in_reference": ignored})
                cases.append(case)
            except Exception as e:  # noqa: BLE001
                skipped.append({"ref": cite, "test": name, "reason": str(e)[:120]})
    return cases, skipped


def extract_slice_shape_rules(ref_root: str):
    """backend/slice.rs host-only tests of compute_output_shape_helper."""
    path = os.path.join(ref_root, "runtime/src/providers/cuda/backend/slice.rs")
    src = open(path).read()
    out = []
    for name, body, line, _ in split_tests(src):
        m = re.search(r"let\s+shape\s*=\s*(\[[^\]]*\]);", body)
        c = re.search(r"compute_output_shape_helper::<\w+>\(\s*&shape,\s*(.+?),\s*&mut out\)", body, re.S)
        if not m or not c:
            continue
        args = split_args(c.group(1))
        try:
            shape = eval_vec(m.group(1), {})
            axes, starts, ends = (eval_vec(a, {}) for a in args[:3])
            steps = None if args[3].strip() == "None" else eval_vec(re.sub(r"^Some\((.*)\)$", r"\1", args[3].strip()), {})
        except Exception:
            continue
        e = re.search(r"assert_eq!\(out,\s*(?:vec!)?(\[[^\]]*\])\)", body)
        out.append({"ref": f"runtime/src/providers/cuda/backend/slice.rs:{line}", "test": name,
                    "shape": shape, "axes": axes, "starts": starts, "ends": ends, "steps": steps,
                    "expected_shape": eval_vec(e.group(1), {}) if e else None,
                    "expect_error": ".unwrap_err()" in body or "panics" in name})
    return out


def extract_kernel_helpers(ref_root: str):
    """cuda/src/kernels tests that drive a helper with literal arguments."""
    out = {}
    base = os.path.join(ref_root, "cuda/src/kernels")
    # reduce_mean: run_reduce_mean_test(shape, data, out_shape, axes, expected)
    src = open(os.path.join(base, "reduce_mean.rs")).read()
    rm = []
    for name, body, line, _ in split_tests(src):
        m = re.search(r"run_reduce_mean_test\(", body)
        if not m:
            continue
        close = matching(body, m.end() - 1)
        a = split_args(body[m.end():close])
        try:
            rm.append({"ref": f"cuda/src/kernels/reduce_mean.rs:{line}", "test": name,
                       "shape": eval_vec(a[0], {}), "data": jsonable(eval_vec(a[1], {})),
                       "out_shape": eval_vec(a[2], {}), "axes": eval_vec(a[3], {}),
                       "expected": jsonable(eval_vec(a[4], {}))})
        except Exception:
            pass
    out["reduce_mean"] = rm
    return out


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    cases, skipped = extract_provider(ref_root)
    doc = {
        "source": "unit tests of kckeiks/rmlk (paths relative to the reference root)",
        "provider_cases": cases,
        "slice_shape_rules": extract_slice_shape_rules(ref_root),
        "kernel_cases": extract_kernel_helpers(ref_root),
        "skipped": skipped,
    }
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "reference_cases.json"), "w") as f:
        json.dump(doc, f, indent=1, sort_keys=True)
    by_op = {}
    for c in cases:
        by_op[c["op"]] = by_op.get(c["op"], 0) + 1
    print(f"{len(cases)} provider cases, {len(doc['slice_shape_rules'])} slice shape rules, "
          f"{sum(len(v) for v in doc['kernel_cases'].values())} kernel helper cases, "
          f"{len(skipped)} skipped")
    print(by_op)
    for s in skipped:
        print("  skipped", s["ref"], s["test"], "--", s["reason"])


if __name__ == "__main__":
    main()

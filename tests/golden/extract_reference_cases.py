#!/usr/bin/env python3
"""Extracts the known-answer vectors the reference's own unit tests hold for the operator path
into tests/golden/reference_cases.json (data only: inputs, attributes, expected outputs).

Run in the build container (the reference tree is not available on the GPU box):

    python tests/golden/extract_reference_cases.py /root/reference

Sources:
  runtime/src/providers/cuda/backend/<op>.rs   #[cfg(test)] OpTest chains (one-op graphs)
      -> "provider_cases", "slice_shape_rules", "skipped"
  cuda/src/kernels/<op>.rs                     the kernel crate's own #[test]s -> "kernel_cases":
      reduce_mean (run_reduce_mean_test), binary (add sub mul div equal greater), pow (run_test, every
      element-type pair the crate tests), where, unary (sqrt neg sin cos sigmoid), cast (the
      generate_cast_test! invocations and the f64 -> f32 overflow test), expand, transpose, trilu,
      scatter_nd, slice, gemm; bodies that are not literal data -> "kernel_skipped"

The Rust test bodies are read as text and only their literals are evaluated: shapes, data vectors,
attributes and the expected vectors of assert_eq! / assert_close / assert_close_eps. Cases whose
body uses anything else are listed under "skipped" / "kernel_skipped" with the reason, so the count
is auditable. One expectation is a formula rather than a literal and is evaluated here: the sigmoid
tests compare with the test module's own `1/(1+exp(-x))` (marked "expected_from" in the case).
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


RUST_DEFAULT = {"float": "float64", "int": "int32"}      # what rustc infers for bare literals

F32_CONSTS = {"PI": math.pi, "FRAC_PI_2": math.pi / 2, "FRAC_PI_3": math.pi / 3,
              "FRAC_PI_4": math.pi / 4, "FRAC_PI_6": math.pi / 6,
              "FRAC_1_SQRT_2": 1 / math.sqrt(2)}


def f32_round(v: float) -> float:
    import numpy as np
    return float(np.float32(v))


def eval_kernel_expr(expr: str, env: dict):
    """eval_vec plus the forms the kernel-crate tests use: `(a..b).collect()`, `x.clone()`,
    `vec![v; x.len()]`, `consts::NAME` (std::f32::consts, rounded to f32)."""
    e = expr.strip()
    if e.startswith("&"):
        e = e[1:].strip()
    if e in env:
        return list(env[e])
    m = re.fullmatch(r"(\w+)\.clone\(\)", e)
    if m and m.group(1) in env:
        return list(env[m.group(1)])
    m = re.fullmatch(r"\(\s*(-?\d+)\s*\.\.\s*(-?\d+)\s*\)\s*\.collect(?:::<[^>]*>)?\(\)", e)
    if m:
        return list(range(int(m.group(1)), int(m.group(2))))
    m = re.fullmatch(r"(?:vec!)?\s*\[\s*([-\d.]+)\s*;\s*(\w+)\.len\(\)\s*\]", e)
    if m and m.group(2) in env:
        return [eval(m.group(1), {"__builtins__": {}}, {})] * len(env[m.group(2)])
    if "consts::" in e:
        e = re.sub(r"(?:std::f32::)?consts::(\w+)", lambda c: repr(f32_round(F32_CONSTS[c.group(1)])), e)
        return [f32_round(v) for v in eval_vec(e, {})]
    return eval_vec(e, env)


def declared_dtype(ty: str | None, expr: str):
    """Element type of a `let` binding: its annotation, a literal suffix, or rustc's default."""
    if ty:
        m = re.search(r"(?:Vec<|&\[|\[)\s*(\w+)", ty)
        if m and m.group(1) in RUST_TYPES:
            return RUST_TYPES[m.group(1)]
    lit = literal_dtype(expr)
    if lit:
        return lit
    m = re.search(r"as\s+(f32|f64|i32|i64)\b", expr)
    if m:
        return RUST_TYPES[m.group(1)]
    return None


def default_dtype(vals):
    if vals and all(isinstance(v, bool) for v in vals):
        return "bool"
    if any(isinstance(v, (float, str)) for v in vals):
        return RUST_DEFAULT["float"]
    return RUST_DEFAULT["int"]


def strip_comments(src: str) -> str:
    return re.sub(r"//[^\n]*", "", src)


def let_statements(body: str):
    """(name, type annotation or None, right side) of every immutable `let` (a `let mut` vector is
    filled by code further down, so its initialiser is not the data), the statement ending at the
    first `;` outside brackets (so `[f32; 1]` and `vec![0.0; n]` stay whole)."""
    for m in re.finditer(r"\blet\s+(?!mut\b)(\w+)\s*", body):
        i, depth, eq = m.end(), 0, None
        while i < len(body):
            ch = body[i]
            if ch in "([{":
                depth += 1
            elif ch in ")]}":
                depth -= 1
            elif ch == "=" and depth == 0 and eq is None and body[i + 1] != "=":
                eq = i
            elif ch == ";" and depth == 0:
                break
            i += 1
        if eq is None:
            continue
        ty = body[m.end():eq].strip()
        yield m.group(1), (ty[1:].strip() if ty.startswith(":") else None), body[eq + 1:i].strip()


def let_bindings(body: str):
    """name -> (values, dtype or None) for every `let` whose right side is literal data."""
    env, types = {}, {}
    for name, ty, expr in let_statements(strip_comments(body)):
        try:
            env[name] = eval_kernel_expr(expr, env)
        except Exception:
            continue
        src = expr.strip().lstrip("&")
        src = src[:-8] if src.endswith(".clone()") else src
        types[name] = declared_dtype(ty, expr) or types.get(src)
    return env, types


# The slice kernel takes the output shape from its caller and only resolves where each output element
# comes from (element i of a dim is input element start + i * step). Three kernel tests hand it a
# shape that the reference's own provider rule (backend/slice.rs:417-452) and ONNX would not
# produce; those cases keep the kernel test's expectation and carry the operator-level one beside it.
SLICE_ONNX_SIDE = {
    # start 10 -> 4, end -1 -> 4, step -1: an EMPTY slice for the operator, the test asks for one element
    "test_overlarge_start_negative_step": {"onnx_output_shape": [0], "onnx_expected": []},
    # ends [3, 4] of a [3, 4] input keep columns 1..3; the tests ask for two columns
    "test_null_axes_and_steps": {"onnx_output_shape": [2, 3],
                                 "onnx_expected": [5.0, 6.0, 7.0, 9.0, 10.0, 11.0]},
    "test_null_steps": {"onnx_output_shape": [2, 3],
                        "onnx_expected": [5.0, 6.0, 7.0, 9.0, 10.0, 11.0]},
}

KERNEL_SUFFIX = {"F16": "float16", "F32": "float32", "F64": "float64", "I8": "int8", "I16": "int16",
                 "I32": "int32", "I64": "int64", "U8": "uint8", "U16": "uint16", "U32": "uint32",
                 "U64": "uint64", "Bool": "bool"}


def kernel_variant_dtype(expr: str):
    """`TransposeKernel::FwdI32` / `SliceKernel::FwdF32WithIndexI64` -> data element type."""
    m = re.search(r"Kernel::\w*?Fwd(F16|F32|F64|I8|I16|I32|I64|U8|U16|U32|U64)", expr)
    return KERNEL_SUFFIX[m.group(1)] if m else None


def call_args(body: str, fn: str):
    m = re.search(fn + r"(?:::<[^>]*>)?\(", body)
    if not m:
        return None
    close = matching(body, m.end() - 1)
    return split_args(body[m.end():close])


def expected_of(body: str, env: dict, result_names=("out", "result")):
    """The vector an `assert_eq!(<result>, X)` / `assert_eq!(X, <result>)` compares with."""
    for m in re.finditer(r"assert_eq!\(", body):
        close = matching(body, m.end() - 1)
        a = split_args(body[m.end():close])
        if len(a) < 2:
            continue
        l, r = a[0].strip().lstrip("&"), a[1].strip().lstrip("&")
        if l in result_names:
            return eval_kernel_expr(r, env)
        if r in result_names:
            return eval_kernel_expr(l, env)
    return None


def htod_vectors(body: str):
    """The literal vectors uploaded with `clone_htod(&vec![..])`, in source order."""
    out = []
    for m in re.finditer(r"clone_htod\(\s*&\s*vec!\s*\[", body):
        open_idx = body.index("[", m.start())
        close = matching(body, open_idx, "[", "]")
        out.append(eval_kernel_expr("vec![" + body[open_idx + 1:close] + "]", {}))
    return out


def relative_epsilon(body: str):
    m = re.search(r"assert_(relative|abs_diff)_eq!\([^;]*?epsilon\s*=\s*([-\deE.]+)", body, re.S)
    return (m.group(1), float(m.group(2))) if m else None


def extract_kernel_helpers(ref_root: str):
    """Known-answer tests of cuda/src/kernels/*.rs. Returns (cases per file, skipped list)."""
    base = os.path.join(ref_root, "cuda/src/kernels")
    out, skipped = {}, []

    def tests_of(fname):
        src = open(os.path.join(base, fname + ".rs")).read()
        for name, body, line, _ in split_tests(src):
            yield name, body, f"cuda/src/kernels/{fname}.rs:{line}", src

    def skip(cite, name, reason):
        skipped.append({"ref": cite, "test": name, "reason": reason})

    # reduce_mean: run_reduce_mean_test(shape, data, out_shape, axes, expected)
    rm = []
    for name, body, cite, _ in tests_of("reduce_mean"):
        a = call_args(body, "run_reduce_mean_test")
        if not a:
            continue
        try:
            rm.append({"ref": cite, "test": name,
                       "shape": eval_vec(a[0], {}), "data": jsonable(eval_vec(a[1], {})),
                       "out_shape": eval_vec(a[2], {}), "axes": eval_vec(a[3], {}),
                       "expected": jsonable(eval_vec(a[4], {}))})
        except Exception as e:  # noqa: BLE001
            skip(cite, name, str(e)[:120])
    out["reduce_mean"] = rm

    # add sub mul div equal greater: two uploaded operands of one shape, one expected vector
    binary = []
    for fname in ("add", "sub", "mul", "div", "equal", "greater"):
        for name, body, cite, _ in tests_of(fname):
            try:
                env, _ = let_bindings(body)
                vecs = htod_vectors(body)
                exp = expected_of(body, env) or env.get("expected")
                if len(vecs) < 2 or exp is None:
                    raise Unparsed("operands or expectation not literal")
                eps = relative_epsilon(body)
                binary.append({"ref": cite, "test": f"{fname}_{name}", "op": fname,
                               "dtype": "float32", "shape": env["output_shape"],
                               "a": jsonable(vecs[0]), "b": jsonable(vecs[1]),
                               "expected": jsonable(exp),
                               "compare": eps[0] if eps else "exact",
                               "epsilon": eps[1] if eps else 0.0})
            except Exception as e:  # noqa: BLE001
                skip(cite, name, str(e)[:120])
    out["binary"] = binary

    # pow: run_test(PowKernel::PowFwd<X><Y>, &shape, &a, &b) with typed a, b, expected
    pw = []
    for name, body, cite, _ in tests_of("pow"):
        try:
            env, types = let_bindings(body)
            a = call_args(body, "run_test")
            if not a:
                raise Unparsed("no run_test call")
            eps = relative_epsilon(body)
            pw.append({"ref": cite, "test": name, "shape": env["shape"],
                       "a": jsonable(env["a"]), "a_dtype": types["a"],
                       "b": jsonable(env["b"]), "b_dtype": types["b"],
                       "expected": jsonable(env["expected"]),
                       "compare": eps[0] if eps else "exact",
                       "epsilon": eps[1] if eps else 0.0})
        except Exception as e:  # noqa: BLE001
            skip(cite, name, str(e)[:120])
    out["pow"] = pw

    # whereop: x, y, cond uploaded in that order
    wh = []
    for name, body, cite, _ in tests_of("whereop"):
        try:
            env, _ = let_bindings(body)
            vecs = htod_vectors(body)
            exp = expected_of(body, env)
            if len(vecs) != 3 or exp is None:
                raise Unparsed("operands or expectation not literal")
            wh.append({"ref": cite, "test": name, "dtype": "float32", "shape": env["output_shape"],
                       "x": jsonable(vecs[0]), "y": jsonable(vecs[1]), "cond": vecs[2],
                       "expected": jsonable(exp)})
        except Exception as e:  # noqa: BLE001
            skip(cite, name, str(e)[:120])
    out["where"] = wh

    # sqrt neg sin cos: one uploaded operand; sigmoid: run_sigmoid_test(&input, shape, stride, &expected)
    un = []
    for fname in ("sqrt", "neg", "sin", "cos"):
        for name, body, cite, _ in tests_of(fname):
            try:
                env, _ = let_bindings(body)
                vecs = htod_vectors(body)
                exp = expected_of(body, env)
                if exp is None and "expected" in env:
                    exp = env["expected"]
                if len(vecs) != 1 or exp is None:
                    raise Unparsed("operand or expectation not literal")
                eps = relative_epsilon(body)
                un.append({"ref": cite, "test": f"{fname}_{name}", "op": fname, "dtype": "float32",
                           "input": jsonable([f32_round(v) for v in vecs[0]]),
                           "expected": jsonable([f32_round(v) for v in exp]),
                           "compare": eps[0] if eps else "exact",
                           "epsilon": eps[1] if eps else 0.0})
            except Exception as e:  # noqa: BLE001
                skip(cite, name, str(e)[:120])
    for name, body, cite, src in tests_of("sigmoid"):
        try:
            env, _ = let_bindings(body)
            if not re.search(r"fn sigmoid\(x: f32\) -> f32 \{\s*1\.0 / \(1\.0 \+ \(-x\)\.exp\(\)\)\s*\}", src):
                raise Unparsed("expectation formula changed")
            if not re.search(r"input\.iter\(\)\.map\(\|&x\| sigmoid\(x\)\)", body):
                raise Unparsed("expectation is not the module's sigmoid formula")
            import numpy as np
            x = np.array(env["input"], dtype=np.float32)
            with np.errstate(over="ignore"):
                exp = (np.float32(1) / (np.float32(1) + np.exp(-x))).astype(np.float32)
            un.append({"ref": cite, "test": name, "op": "sigmoid", "dtype": "float32",
                       "input": jsonable([float(v) for v in x]),
                       "expected": jsonable([float(v) for v in exp]),
                       "expected_from": "the test module's own formula 1/(1+exp(-x)) in f32 "
                                        "(cuda/src/kernels/sigmoid.rs:37-39), evaluated by the extractor",
                       "shape": env["shape"], "compare": "abs_diff", "epsilon": 1e-6})
        except Exception as e:  # noqa: BLE001
            skip(cite, name, str(e)[:120])
    out["unary"] = un

    # cast: generate_cast_test!(name, CastKernel::XToY, in_ty, out_ty, [inputs], [expected])
    ct = []
    src = open(os.path.join(base, "cast.rs")).read()
    for m in re.finditer(r"generate_cast_test!\(\s*test_", src):
        open_idx = src.index("(", m.start())
        close = matching(src, open_idx)
        a = split_args(strip_comments(src[open_idx + 1:close]))
        line = src.count("\n", 0, m.start()) + 1
        cite = f"cuda/src/kernels/cast.rs:{line}"
        try:
            ct.append({"ref": cite, "test": a[0], "src_dtype": RUST_TYPES[a[2]],
                       "dst_dtype": RUST_TYPES[a[3]], "input": jsonable(eval_vec(a[4], {})),
                       "expected": jsonable(eval_vec(a[5], {}))})
        except Exception as e:  # noqa: BLE001
            skip(cite, a[0], str(e)[:120])
    for name, body, cite, _ in tests_of("cast"):
        if name == "test_cast_f64_to_f32_inf":
            vecs = htod_vectors(body)
            checks = re.findall(r"assert(?:_eq)?!\(result\[(\d)\](?:\.is_(nan)\(\)|,\s*([^)]+))\)", body)
            exp = [None] * len(vecs[0])
            for i, nan, val in checks:
                exp[int(i)] = float("nan") if nan else eval_vec("[" + val + "]", {})[0]
            ct.append({"ref": cite, "test": name, "src_dtype": "float64", "dst_dtype": "float32",
                       "input": jsonable(vecs[0]), "expected": jsonable(exp)})
    out["cast"] = ct

    # expand: launch_expand_test(&input, input_shape, output_shape, ExpandKernel::Fwd<T>)
    ex = []
    for name, body, cite, _ in tests_of("expand"):
        try:
            env, types = let_bindings(body)
            a = call_args(body, "launch_expand_test")
            exp = expected_of(body, env)
            if exp is None and re.search(r"assert_eq!\(result\.len\(\),\s*0\)", body):
                exp = []
            if exp is None:
                raise Unparsed("expectation built by loops, not a literal")
            ex.append({"ref": cite, "test": name, "dtype": kernel_variant_dtype(a[3]),
                       "input": jsonable(env["input"]), "input_shape": env["input_shape"],
                       "output_shape": env["output_shape"], "expected": jsonable(exp)})
        except Exception as e:  # noqa: BLE001
            skip(cite, name, str(e)[:120])
    out["expand"] = ex

    # transpose: launch_transpose_test(&input, shape, perm, TransposeKernel::Fwd<T>); the element
    # type is the HOST vector's (an i32 vector through the 4-byte FwdF32 kernel stays i32)
    tr = []
    for name, body, cite, _ in tests_of("transpose"):
        try:
            env, types = let_bindings(body)
            a = call_args(body, "launch_transpose_test")
            shape = eval_kernel_expr(a[1], env)
            perm = eval_kernel_expr(a[2], env)
            dt = types.get("input") or default_dtype(env["input"])
            case = {"ref": cite, "test": name, "dtype": dt, "input": jsonable(env["input"]),
                    "input_shape": shape, "perm": perm}
            if "#[should_panic]" in open(os.path.join(base, "transpose.rs")).read().split("fn " + name)[0][-40:]:
                case["expect_error"] = True
            else:
                exp = expected_of(body, env)
                if exp is None and re.search(r"assert!\(out\.is_empty\(\)\)", body):
                    exp = []
                if exp is None:
                    raise Unparsed("expectation built by loops, not a literal")
                case["expected"] = jsonable(exp)
            tr.append(case)
        except Exception as e:  # noqa: BLE001
            skip(cite, name, str(e)[:120])
    out["transpose"] = tr

    # trilu: launch_trilu_test(TriluKernel::Fwd<T>, &input, &shape, upper, k)
    tl = []
    for name, body, cite, _ in tests_of("trilu"):
        try:
            env, types = let_bindings(body)
            a = call_args(body, "launch_trilu_test")
            tl.append({"ref": cite, "test": name, "dtype": kernel_variant_dtype(a[0]),
                       "input": jsonable(env["input"]), "shape": env["shape"],
                       "upper": a[3].strip() == "true", "k": int(a[4]),
                       "expected": jsonable(env["expected"])})
        except Exception as e:  # noqa: BLE001
            skip(cite, name, str(e)[:120])
    out["trilu"] = tl

    # scatter_nd: run_scatter_nd_test(data_shape, indices_shape, indices, updates_shape, updates,
    # expected) over zero-filled f32 data. The kernel reads rank-1 indices as one-element tuples
    # (scatter_nd.rs: `num_idx_tuples = if indices_rank == 1 { product }`), which ONNX would write
    # as shape [n, 1]: such cases are recorded with that shape and `indices_shape_in_reference`.
    sc = []
    for name, body, cite, _ in tests_of("scatter_nd"):
        try:
            env, _ = let_bindings(body)
            if not call_args(body, "run_scatter_nd_test"):
                raise Unparsed("no run_scatter_nd_test call")
            ishape = env["indices_shape"]
            case = {"ref": cite, "test": name, "dtype": "float32", "data_shape": env["data_shape"],
                    "indices_shape": ishape if len(ishape) > 1 else ishape + [1],
                    "indices": env["indices_data"], "updates_shape": env["updates_shape"],
                    "updates": jsonable(env["updates_data"]),
                    "expected": jsonable(env["expected_output"])}
            if len(ishape) == 1:
                case["indices_shape_in_reference"] = ishape
            sc.append(case)
        except Exception as e:  # noqa: BLE001
            skip(cite, name, str(e)[:120])
    out["scatter_nd"] = sc

    # slice: launch_slice_test::<T, Tind>(&input, input_shape, output_shape, starts, ends, axes,
    # steps, kernel); empty axes / steps are the ONNX "absent" inputs
    sl = []
    for name, body, cite, _ in tests_of("slice"):
        try:
            env, types = let_bindings(body)
            a = call_args(body, "launch_slice_test")
            exp = expected_of(body, env)
            if exp is None:
                raise Unparsed("expectation not a literal")
            if name in SLICE_ONNX_SIDE:
                onnx_side = SLICE_ONNX_SIDE[name]
            else:
                onnx_side = {}
            sl.append({**onnx_side, "ref": cite, "test": name, "dtype": kernel_variant_dtype(a[7]),
                       "input": jsonable(env["input"]), "input_shape": env["input_shape"],
                       "output_shape": env["output_shape"], "starts": env["starts"],
                       "ends": env["ends"], "axes": env["axes"], "steps": env["steps"],
                       "expected": jsonable(exp)})
        except Exception as e:  # noqa: BLE001
            skip(cite, name, str(e)[:120])
    out["slice"] = sl

    # gemm: [1,2,2] x [1,2,2] through gemm_params / strided_batch_config
    gm = []
    for name, body, cite, _ in tests_of("gemm"):
        try:
            env, _ = let_bindings(body)
            vecs = htod_vectors(body)
            exp = expected_of(body, env)
            a = call_args(body, "gemm_params")
            gm.append({"ref": cite, "test": name, "dtype": "float32", "lhs_shape": env["lhs_shape"],
                       "rhs_shape": env["rhs_shape"], "lhs": jsonable(vecs[0]),
                       "rhs": jsonable(vecs[1]), "trans_a": a[4].strip() == "true",
                       "trans_b": a[5].strip() == "true", "expected": jsonable(exp)})
        except Exception as e:  # noqa: BLE001
            skip(cite, name, str(e)[:120])
    out["gemm"] = gm
    return out, skipped


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    cases, skipped = extract_provider(ref_root)
    kernel_cases, kernel_skipped = extract_kernel_helpers(ref_root)
    doc = {
        "source": "unit tests of kckeiks/rmlk (paths relative to the reference root)",
        "provider_cases": cases,
        "slice_shape_rules": extract_slice_shape_rules(ref_root),
        "kernel_cases": kernel_cases,
        "kernel_skipped": kernel_skipped,
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
    print({k: len(v) for k, v in doc["kernel_cases"].items()})
    for s in kernel_skipped:
        print("  skipped", s["ref"], s["test"], "--", s["reason"])
    for s in skipped:
        print("  skipped", s["ref"], s["test"], "--", s["reason"])


if __name__ == "__main__":
    main()

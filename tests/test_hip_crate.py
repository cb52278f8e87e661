"""The Rust crate under hip/ binds the C ABI of include/rmlk_hip.h: its ffi.rs is generated from the
header and must be up to date, and the constants and structs written out by hand in the generator
must agree with the header. (There is no Rust toolchain here: the crate itself is not compiled.)"""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rmlk_hip.h")
FFI = os.path.join(ROOT, "hip", "src", "ffi.rs")


def _header():
    with open(HEADER) as f:
        return re.sub(r"/\*.*?\*/", " ", f.read(), flags=re.S)


def test_ffi_rs_is_what_the_generator_writes():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "hip", "gen_ffi.py"), "--check"])
    assert r.returncode == 0, "hip/src/ffi.rs is out of date: run python hip/gen_ffi.py"


def test_every_entry_point_is_bound_with_its_argument_count():
    protos = dict()
    for stmt in re.split(r"[;{}]", _header()):
        m = re.search(r"(rmlk_hip_\w+)\s*\(([^()]*)\)\s*$", stmt, flags=re.S)
        if m:
            params = m.group(2).strip()
            protos[m.group(1)] = 0 if params in ("", "void") else params.count(",") + 1
    assert len(protos) >= 59
    with open(FFI) as f:
        ffi = f.read()
    bound = dict()
    for m in re.finditer(r"pub fn (rmlk_hip_\w+)\(([^)]*)\)", ffi, flags=re.S):
        args = [a for a in m.group(2).split(",") if a.strip()]
        bound[m.group(1)] = len(args)
    assert bound == protos


def test_constants_agree_with_the_header():
    hdr = _header()
    with open(FFI) as f:
        ffi = f.read()
    enums = dict((m.group(1), int(m.group(2))) for m in re.finditer(r"\b(RMLK_[A-Z0-9_]+)\s*=\s*(-?\d+)", hdr))
    assert len(enums) >= 38
    consts = dict((m.group(1), int(m.group(2))) for m in re.finditer(r"pub const (RMLK_[A-Z0-9_]+): i32 = (-?\d+);", ffi))
    assert consts == enums
    assert "pub const RMLK_MAX_RANK: usize = 8;" in ffi and re.search(r"#define RMLK_MAX_RANK 8\b", hdr)


def test_structs_list_the_header_fields_in_order():
    hdr = _header()
    with open(FFI) as f:
        ffi = f.read()
    for name in ("rmlk_dims", "rmlk_row_stream", "rmlk_device_info"):
        c_body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (name, name), hdr, flags=re.S).group(1)
        c_fields = [re.search(r"(\w+)(\[[^\]]*\])?$", d.strip()).group(1) for d in c_body.split(";") if d.strip()]
        r_body = re.search(r"pub struct %s \{(.*?)\n\}" % name, ffi, flags=re.S).group(1)
        r_fields = re.findall(r"pub (\w+):", r_body)
        assert r_fields == c_fields, name


def test_kernel_modules_exist_for_the_reference_layout():
    with open(os.path.join(ROOT, "hip", "src", "kernels", "mod.rs")) as f:
        mods = re.findall(r"pub mod (\w+);", f.read())
    for m in mods:
        assert os.path.isfile(os.path.join(ROOT, "hip", "src", "kernels", m + ".rs")), m
    # the operators of the decoder path, by the reference's module names (cuda/src/kernels/mod.rs)
    for m in ("add", "sub", "mul", "div", "pow", "equal", "greater", "binary", "unary", "neg", "sqrt", "sin", "cos",
              "sigmoid", "cast", "expand", "gemm", "reduce_mean", "scatter_nd", "slice", "softmax", "transpose",
              "trilu", "whereop"):
        assert m in mods, m


def _call_sites():
    """(entry point, number of arguments, file) of every `ffi::rmlk_hip_*( .. )` call under hip/src."""
    out = []
    src_dir = os.path.join(ROOT, "hip", "src")
    for base, _, files in os.walk(src_dir):
        for fn in files:
            if not fn.endswith(".rs") or fn == "ffi.rs":
                continue
            text = open(os.path.join(base, fn)).read()
            text = re.sub(r"//[^\n]*", "", text)
            for m in re.finditer(r"ffi::(rmlk_hip_\w+)\s*\(", text):
                depth, i, args, cur = 1, m.end(), [], ""
                while depth and i < len(text):
                    ch = text[i]
                    if ch in "([{":
                        depth += 1
                    elif ch in ")]}":
                        depth -= 1
                        if depth == 0:
                            break
                    if ch == "," and depth == 1:
                        args.append(cur)
                        cur = ""
                    else:
                        cur += ch
                    i += 1
                if cur.strip():
                    args.append(cur)
                out.append((m.group(1), len(args), os.path.relpath(os.path.join(base, fn), ROOT)))
    return out


def _bound():
    with open(FFI) as f:
        ffi = f.read()
    return {m.group(1): len([a for a in m.group(2).split(",") if a.strip()])
            for m in re.finditer(r"pub fn (rmlk_hip_\w+)\(([^)]*)\)", ffi, flags=re.S)}


def test_every_call_site_passes_the_declared_number_of_arguments():
    """The crate cannot be compiled here; this is the part of the compiler's job that text can do."""
    bound = _bound()
    sites = _call_sites()
    assert len(sites) >= 45
    wrong = [(name, n, bound.get(name), path) for name, n, path in sites if bound.get(name) != n]
    assert not wrong, wrong


def test_entry_points_the_reference_backends_need_are_wrapped():
    """Operators of the reference whose backends have no kernel-crate module (they move or build data
    through cudarc: backend/reshape.rs:46, constant_of_shape.rs:59-62, range.rs:140-151, shape.rs:67-72,
    concat.rs:28-76) still need these entry points from the Rust side."""
    called = {name for name, _, _ in _call_sites()}
    for need in ("rmlk_hip_fill", "rmlk_hip_range", "rmlk_hip_memcpy_dtod", "rmlk_hip_concat",
                 "rmlk_hip_concat_many", "rmlk_hip_device_info", "rmlk_hip_write_small", "rmlk_hip_memset",
                 "rmlk_hip_malloc", "rmlk_hip_free", "rmlk_hip_memcpy_htod", "rmlk_hip_memcpy_dtoh",
                 "rmlk_hip_stream_sync", "rmlk_hip_status_string"):
        assert need in called, need
    # one wrapper per kernel row of the operator path
    for need in ("rmlk_hip_binary", "rmlk_hip_where", "rmlk_hip_unary", "rmlk_hip_cast", "rmlk_hip_reduce_mean",
                 "rmlk_hip_softmax", "rmlk_hip_matmul", "rmlk_hip_transpose", "rmlk_hip_expand", "rmlk_hip_slice",
                 "rmlk_hip_gather", "rmlk_hip_scatter_nd", "rmlk_hip_trilu"):
        assert need in called, need

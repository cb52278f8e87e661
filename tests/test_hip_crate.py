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

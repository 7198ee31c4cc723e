"""The Rust binding under rust/ against include/descent_hip.h, mechanically (no Rust toolchain exists here, so the
files cannot be compiled): every struct of the header has a #[repr(C)] struct of the same name with the same fields
in the same order and matching types; the layout those Rust declarations imply (computed with the repr(C) rules)
equals what gcc reports for the header with sizeof/offsetof, and what the ctypes mirror in descent_amd/_abi.py has;
every exported function has an `extern "C"` line with the same parameter names and matching types; every constant
of the kinds the marshalling code uses has the header's value."""
import ctypes as C
import os
import re
import shutil
import subprocess

import pytest

from descent_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "descent_hip.h")
HIP_RS = os.path.join(ROOT, "rust", "src", "device", "hip.rs")
MARSHAL_RS = os.path.join(ROOT, "rust", "src", "kernel_marshal.rs")

C_TO_RUST = {
    "int32_t": "i32", "int64_t": "i64", "uint32_t": "u32", "uint64_t": "u64", "size_t": "usize", "int": "c_int",
    "char": "c_char", "double": "f64", "void": "c_void", "dsc_buf": "dsc_buf",
}
RUST_SCALARS = {"i32": (4, 4), "u32": (4, 4), "i64": (8, 8), "u64": (8, 8), "usize": (8, 8), "c_char": (1, 1), "c_int": (4, 4),
                "f64": (8, 8), "dsc_buf": (8, 8)}


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def _c_type_to_rust(ctype):
    """'const dsc_view*' -> '*const dsc_view', 'dsc_ctx**' -> '*mut *mut dsc_ctx', 'int32_t' -> 'i32'."""
    ctype = ctype.strip()
    stars = ctype.count("*")
    base = ctype.replace("*", "").strip()
    const = base.startswith("const ")
    base = base.replace("const ", "").replace("struct ", "").strip()
    rust = C_TO_RUST.get(base, base)
    for i in range(stars):
        rust = ("*const " if (const and i == 0) else "*mut ") + rust
    return rust


def header_structs():
    text = _strip_comments(open(HEADER).read())
    out = {}
    for body, name in re.findall(r"typedef struct \w+ \{(.*?)\}\s*(\w+);", text, re.S):
        fields = []
        for decl in body.split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            m = re.match(r"(.+?)\s*(\w+)(?:\[(\w+)\])?$", decl)
            ctype, fname, count = m.group(1), m.group(2), m.group(3)
            rust = _c_type_to_rust(ctype)
            if count:
                rust = f"[{rust}; {count}]"
            fields.append((fname, rust))
        out[name] = fields
    return out


def rust_structs():
    text = _strip_comments(open(HIP_RS).read())
    out = {}
    for attrs, name, body in re.findall(r"((?:#\[[^\]]*\]\s*)+)pub struct (\w+) \{(.*?)\}", text, re.S):
        if "repr(C)" not in attrs:
            continue
        fields = []
        for decl in body.split(",\n"):
            decl = " ".join(decl.split()).rstrip(",")
            if not decl:
                continue
            m = re.match(r"(?:pub )?(\w+): (.+)$", decl)
            fields.append((m.group(1), m.group(2)))
        out[name] = fields
    return out


def header_functions():
    text = _strip_comments(open(HEADER).read())
    out = {}
    for ret, name, args in re.findall(r"^\s*(int|int64_t|void|const char\*)\s+(dsc_\w+)\s*\(([^)]*)\)\s*;", text, re.M):
        params = []
        for a in args.split(","):
            a = " ".join(a.split())
            if a in ("void", ""):
                continue
            m = re.match(r"(.+?)\s*(\w+)$", a)
            params.append((m.group(2), _c_type_to_rust(m.group(1))))
        out[name] = (None if ret == "void" else _c_type_to_rust(ret), params)
    return out


def rust_functions():
    text = _strip_comments(open(HIP_RS).read())
    block = re.search(r'extern "C" \{(.*?)\n\}', text, re.S).group(1)
    out = {}
    for name, args, ret in re.findall(r"pub fn (dsc_\w+)\(([^)]*)\)(?: -> ([^;]+))?;", block):
        params = []
        for a in args.split(","):
            a = " ".join(a.split())
            if a:
                pname, ptype = a.split(": ", 1)
                params.append((pname, ptype))
        out[name] = (ret.strip() if ret else None, params)
    return out


def test_every_header_struct_has_a_field_for_field_rust_mirror():
    hs, rs = header_structs(), rust_structs()
    assert set(hs) == {"dsc_shape", "dsc_view", "dsc_pe_op", "dsc_kernel_desc", "dsc_caps", "dsc_cluster_output", "dsc_cluster",
                       "dsc_param_io", "dsc_schedule_desc"}
    for name, fields in hs.items():
        assert name in rs, f"{name} has no #[repr(C)] struct in hip.rs"
        assert rs[name] == fields, f"{name}: header {fields} != rust {rs[name]}"


def _rust_layout(structs, consts):
    """size, alignment and field offsets that #[repr(C)] gives each struct."""
    done = {}

    def type_layout(t):
        t = t.strip()
        if t.startswith("*"):
            return 8, 8
        m = re.match(r"\[(.+); (\w+)\]$", t)
        if m:
            size, align = type_layout(m.group(1))
            n = consts[m.group(2)] if not m.group(2).isdigit() else int(m.group(2))
            return size * n, align
        if t in RUST_SCALARS:
            return RUST_SCALARS[t]
        return struct_layout(t)[:2]

    def struct_layout(name):
        if name in done:
            return done[name]
        offset, align, offsets = 0, 1, {}
        for fname, ftype in structs[name]:
            size, a = type_layout(ftype)
            offset = (offset + a - 1) // a * a
            offsets[fname] = offset
            offset += size
            align = max(align, a)
        done[name] = ((offset + align - 1) // align * align, align, offsets)
        return done[name]

    return {name: struct_layout(name) for name in structs}


def test_rust_layout_equals_the_c_compilers_and_the_ctypes_mirror(tmp_path):
    gcc = shutil.which("gcc")
    if not gcc:
        pytest.skip("no gcc")
    hs = header_structs()
    rust_text = open(HIP_RS).read()
    consts = {m.group(1): int(m.group(2)) for m in re.finditer(r"pub const (\w+): usize = (\d+);", rust_text)}
    assert consts["DSC_MAX_DIM"] == 7
    rs = rust_structs()
    layout = _rust_layout({name: rs[name] for name in hs}, consts)  # the opaque handle types have no layout to compare
    lines = ['#include "descent_hip.h"', "#include <stddef.h>", "#include <stdio.h>", "int main(void) {"]
    for name, fields in hs.items():
        lines.append(f'    printf("{name} %zu\\n", sizeof({name}));')
        for fname, _ in fields:
            lines.append(f'    printf("{name}.{fname} %zu\\n", offsetof({name}, {fname}));')
    lines += ["    return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "layout"
    subprocess.run([gcc, "-std=c99", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    reported = dict(line.split() for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for name, (size, _, offsets) in layout.items():
        assert int(reported[name]) == size, (name, reported[name], size)
        for fname, off in offsets.items():
            assert int(reported[f"{name}.{fname}"]) == off, (name, fname)
    mirrors = {"dsc_shape": _abi.CShape, "dsc_view": _abi.CView, "dsc_pe_op": _abi.CPeOp, "dsc_kernel_desc": _abi.CKernelDesc,
               "dsc_caps": _abi.CCaps, "dsc_cluster_output": _abi.CClusterOutput, "dsc_cluster": _abi.CCluster,
               "dsc_param_io": _abi.CParamIO, "dsc_schedule_desc": _abi.CScheduleDesc}
    for name, ctype in mirrors.items():
        assert C.sizeof(ctype) == layout[name][0], name
        for fname, off in layout[name][2].items():
            assert getattr(ctype, fname).offset == off, (name, fname)


def test_every_export_has_an_extern_line_with_the_same_signature():
    hf, rf = header_functions(), rust_functions()
    assert len(hf) >= 45
    assert set(hf) == set(rf), (sorted(set(hf) - set(rf)), sorted(set(rf) - set(hf)))
    for name, (ret, params) in hf.items():
        rret, rparams = rf[name]
        assert rret == ret, (name, ret, rret)
        assert rparams == params, (name, params, rparams)


def test_constants_agree_with_the_header():
    header = _strip_comments(open(HEADER).read())
    rust = open(HIP_RS).read()
    # enum members with explicit or running values
    values = {}
    for body in re.findall(r"typedef enum \w+ \{(.*?)\}", header, re.S):
        nxt = 0
        for item in body.split(","):
            item = item.strip()
            if not item:
                continue
            if "=" in item:
                k, v = (s.strip() for s in item.split("="))
                nxt = int(v, 0)
            else:
                k = item
            values[k] = nxt
            nxt += 1
    for m in re.finditer(r"#define (DSC_\w+) \(?(\d+)u?(?: << (\d+))?\)?", header):
        values[m.group(1)] = int(m.group(2)) << int(m.group(3) or 0)
    checked = 0
    for m in re.finditer(r"pub const (DSC_\w+): \w+ = (\d+)(?: << (\d+))?;", rust):
        assert m.group(1) in values, m.group(1)
        assert values[m.group(1)] == int(m.group(2)) << int(m.group(3) or 0), m.group(1)
        checked += 1
    assert checked >= 25
    # the op codes the marshalling writes are positions in the header's enums
    marshal = open(MARSHAL_RS).read()
    for enum_prefix, rust_enum in (("DSC_UN_", "UnaryOp"), ("DSC_BIN_", "BinaryOp"), ("DSC_CMP_", "CompareMode"), ("DSC_REDUCE_", "ReduceOp"),
                                   ("DSC_MATMUL_", "MatMulOutputMode")):
        for variant, code in re.findall(rust_enum + r"::(\w+) => (\d+),", marshal):
            # FloatToUint -> FLOAT_TO_UINT, UBitXor -> UBITXOR, Batches -> BATCHES
            snake = re.sub(r"(?<=[a-z])(?=[A-Z])", "_", variant).upper()
            key = enum_prefix + snake
            if key not in values:
                key = enum_prefix + variant.upper()
            assert values[key] == int(code), (rust_enum, variant, code)

"""The Rust binding (integration/rust/) against the C header it binds.

No Rust toolchain exists in this image, so the binding cannot be compiled here.  What can be checked mechanically is
that `hip_ffi.rs` declares exactly the functions of `include/rt_hip.h` with the same argument names, order and
machine types, that its constants carry the header's values, and that `hip.rs` implements every method of the
reference's `trait Backend` (backend/mod.rs:216-472; the method list below is spelled out here, the reference is
not read at test time).
"""
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "rt_hip.h"
FFI = ROOT / "integration" / "rust" / "hip_ffi.rs"
HIP = ROOT / "integration" / "rust" / "hip.rs"

C_TO_RUST = {
    "rt_ctx*": "*mut rt_ctx",
    "rt_ctx**": "*mut *mut rt_ctx",
    "rt_event*": "*mut rt_event",
    "rt_event**": "*mut *mut rt_event",
    "const void*": "*const c_void",
    "void*": "*mut c_void",
    "void**": "*mut *mut c_void",
    "const uint64_t*": "*const u64",
    "uint64_t*": "*mut u64",
    "const int64_t*": "*const i64",
    "const void*const*": "*const *const c_void",
    "const rt_chain_step*": "*const rt_chain_step",
    "int32_t*": "*mut i32",
    "int64_t*": "*mut i64",
    "float*": "*mut f32",
    "const char*": "*const c_char",
    "int32_t": "i32",
    "int64_t": "i64",
    "uint64_t": "u64",
    "uint32_t": "u32",
}


def strip_c_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def header_functions():
    text = strip_c_comments(HEADER.read_text())
    out = {}
    for m in re.finditer(r"(const\s+char\s*\*|int32_t)\s+(rt_\w+)\s*\(([^)]*)\)\s*;", text):
        ret, name, args = m.group(1), m.group(2), m.group(3).strip()
        params = []
        if args and args != "void":
            for a in args.split(","):
                a = " ".join(a.split())
                pm = re.match(r"(.*?)(\w+)$", a)
                ctype = pm.group(1).replace(" *", "*").replace("* ", "*").strip()
                params.append((pm.group(2), ctype))
        out[name] = (" ".join(ret.split()).replace(" *", "*"), params)
    return out


def rust_functions():
    text = re.sub(r"//[^\n]*", " ", FFI.read_text())
    block = text[text.index('extern "C"'):]
    out = {}
    for m in re.finditer(r"pub fn (rt_\w+)\s*\(([^)]*)\)\s*->\s*([^;]+);", block):
        name, args, ret = m.group(1), m.group(2).strip(), m.group(3).strip()
        params = []
        if args:
            for a in args.split(","):
                a = " ".join(a.split())
                if not a:
                    continue
                pname, ptype = a.split(":", 1)
                params.append((pname.strip(), ptype.strip()))
        out[name] = (ret, params)
    return out


def test_same_functions_in_header_and_binding():
    c, r = header_functions(), rust_functions()
    assert len(c) >= 47, sorted(c)
    assert sorted(c) == sorted(r), (sorted(set(c) - set(r)), sorted(set(r) - set(c)))


@pytest.mark.parametrize("name", sorted(header_functions()))
def test_arguments_agree(name):
    c_ret, c_params = header_functions()[name]
    r_ret, r_params = rust_functions()[name]
    assert C_TO_RUST[c_ret] == r_ret
    assert [p for p, _ in c_params] == [p for p, _ in r_params]
    for (pname, ctype), (_, rtype) in zip(c_params, r_params):
        assert ctype in C_TO_RUST, f"{name}({pname}): C type {ctype!r} has no Rust mapping in this test"
        assert C_TO_RUST[ctype] == rtype, f"{name}({pname}): {ctype} declared as {rtype}"


def test_chain_step_struct_agrees():
    """rt_chain_step crosses the boundary by pointer: same fields, order and machine types on both sides (24 bytes, no padding)."""
    text = strip_c_comments(HEADER.read_text())
    m = re.search(r"typedef\s+struct\s+rt_chain_step\s*\{(.*?)\}\s*rt_chain_step\s*;", text, flags=re.S)
    c_fields = []
    for decl in m.group(1).split(";"):
        decl = " ".join(decl.split())
        if not decl:
            continue
        fm = re.match(r"(\w+) (\w+)(?:\[(\d+)\])?$", decl)
        c_fields.append((fm.group(2), fm.group(1), fm.group(3)))
    rust = re.sub(r"//[^\n]*", " ", FFI.read_text())
    rm = re.search(r"#\[repr\(C\)\]\s*(?:#\[derive\([^)]*\)\]\s*)?pub struct rt_chain_step\s*\{(.*?)\}", rust, flags=re.S)
    r_fields = []
    for decl in rm.group(1).split(","):
        decl = " ".join(decl.split())
        if decl:
            name, ty = decl.replace("pub ", "").split(":")
            r_fields.append((name.strip(), ty.strip()))
    assert [f[0] for f in c_fields] == [f[0] for f in r_fields]
    size = 0
    for (name, ctype, count), (_, rtype) in zip(c_fields, r_fields):
        want = {"int32_t": "i32", "uint8_t": "u8"}[ctype]
        assert rtype == (f"[{want}; {count}]" if count else want), (name, rtype)
        size += {"int32_t": 4, "uint8_t": 1}[ctype] * int(count or 1)
    assert size == 24


def header_constants():
    """Enumerators (with C's implicit +1 numbering) and integer #defines of the header."""
    text = strip_c_comments(HEADER.read_text())
    out = {}
    for m in re.finditer(r"typedef\s+enum\s+\w+\s*\{(.*?)\}", text, flags=re.S):
        nxt = 0
        for item in m.group(1).split(","):
            item = item.strip()
            if not item:
                continue
            if "=" in item:
                k, v = (x.strip() for x in item.split("="))
                nxt = int(v, 0)
            else:
                k = item
            out[k] = nxt
            nxt += 1
    for m in re.finditer(r"#define\s+(RT_\w+)\s+(0x[0-9a-fA-F]+|\d+)u?\s", text):
        out[m.group(1)] = int(m.group(2), 0)
    m = re.search(r"#define\s+RT_STATIC_SCRATCH_BYTES\s+\((\d+)u\s*<<\s*(\d+)\)", text)
    out["RT_STATIC_SCRATCH_BYTES"] = int(m.group(1)) << int(m.group(2))
    return out


def test_constants_agree():
    c = header_constants()
    text = FFI.read_text()
    seen = 0
    for m in re.finditer(r"pub const (RT_\w+): [iu]32 = ([^;]+);", text):
        name, expr = m.group(1), m.group(2).strip()
        value = eval(expr, {"__builtins__": {}})  # integer literals and shifts only
        assert name in c, f"{name} is not in the header"
        assert c[name] == value, f"{name}: header {c[name]}, binding {value}"
        seen += 1
    assert seen >= 60
    for family in ("RT_E_", "RT_U_", "RT_S_"):
        missing = [k for k in c if k.startswith(family) and not k.endswith("COUNT") and f"pub const {k}:" not in text]
        assert not missing, missing


UNARY = ["neg", "relu", "sigmoid", "silu", "tanh", "abs", "sqrt", "ln", "expm1", "ln1p", "floor", "ceil", "round", "trunc",
         "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "asinh", "acosh", "atanh", "rsqrt", "reciprocal",
         "square", "cube", "exp", "sign"]
SCALAR = ["add", "sub", "mul", "div", "log", "log1p", "leaky_relu", "elu"]
PLAIN = ["device_type", "alloc_from_slice", "alloc", "copy_from_slice", "copy_range_within", "read", "write", "len", "copy",
         "dump", "convert", "new", "fill_nd", "fill_1d_strided", "fill_contiguous", "broadcast", "apply_reduce_contiguous_flat",
         "apply_reduce_contiguous_nd", "apply_argmax_contiguous_flat", "apply_argmax_contiguous_nd", "apply_conv_2d"]


def test_every_trait_method_is_implemented():
    text = HIP.read_text()
    body = text[text.index("impl Backend for Hip"):text.index("impl<T: TensorValue> BackendMatMul<T> for Hip")]
    for name in PLAIN:
        assert re.search(rf"\bfn {name}\b", body), name
    # the two macros produce the four methods of each op; each op is invoked once with the header's code of the same name
    for macro, prefix in (("hip_unary", "apply_"), ("hip_scalar", "scalar_apply_")):
        mdef = text[text.index(f"macro_rules! {macro}"):]
        mdef = mdef[:mdef.index("\n}\n")]
        for suffix in ("", "_nd", "_1d_strided", "_contiguous"):
            want = f"[<{prefix} $name {suffix}>]" if suffix else f"[<{prefix} $name>]"
            assert want in mdef, (macro, suffix)
    for name in UNARY:
        assert re.search(rf"hip_unary! \{{{name}, ffi::RT_U_{name.upper()}[,}}]", body), name
    for name in SCALAR:
        assert re.search(rf"hip_scalar! \{{{name}, ffi::RT_S_{name.upper()}[,}}]", body), name
    assert "fn matmul" in text[text.index("BackendMatMul<T> for Hip"):]
    assert "todo!" not in text.replace("never `todo!()`", "") and "unimplemented!" not in text


def test_binding_calls_only_declared_functions():
    declared = set(rust_functions())
    used = set(re.findall(r"ffi::(rt_\w+)\s*\(", HIP.read_text()))
    assert used <= declared, used - declared
    # everything behind the trait is reached
    for name in ("rt_broadcast", "rt_reduce_nd", "rt_reduce_flat", "rt_argmax_nd", "rt_argmax_flat", "rt_unary_nd",
                 "rt_scalar_nd", "rt_fill_nd", "rt_convert", "rt_equal", "rt_matmul", "rt_copy_range_within"):
        assert name in used, name

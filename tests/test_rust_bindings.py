"""Keeps the Rust shim's declarations (bindings/rust/ug-hip/src/ffi.rs) in step with include/ughip.h: the same
functions with the same number and types of arguments and the same return type, the same #[repr(C)] structs field
for field, the same dtype codes.  No Rust toolchain exists here, so this is what stands between the two files and a
silent ABI mismatch."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ughip.h")
RUST = os.path.join(ROOT, "bindings", "rust")
FFI = os.path.join(RUST, "ug-hip", "src", "ffi.rs")

C_TO_RUST_BASE = {"int": "c_int", "unsigned": "c_uint", "size_t": "usize", "float": "f32", "char": "c_char", "void": "c_void",
                  "ughip_device": "UghipDevice", "ughip_slice": "UghipSlice", "ughip_func": "UghipFunc", "ughip_event": "UghipEvent",
                  "ughip_ssa": "UghipSsa", "ughip_func_info": "UghipFuncInfo", "ughip_instr": "UghipInstr", "ughip_kernel_arg": "UghipKernelArg", "ughip_a": "UghipA",
                  "uint8_t": "u8", "uint16_t": "u16", "uint32_t": "u32", "uint64_t": "u64", "int32_t": "i32", "int64_t": "i64"}


def _strip_c(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return text


def c_type_to_rust(ctype):
    """'const ughip_slice* const*' -> '*const *const UghipSlice' (a const before a star makes that pointer *const)."""
    toks = ctype.replace("*", " * ").split()
    const, base, ptrs = False, None, []
    for tok in toks:
        if tok == "const":
            const = True
        elif tok == "*":
            ptrs.append("*const " if const else "*mut ")
            const = False
        else:
            assert base is None, ctype
            base = C_TO_RUST_BASE[tok]
    if const and ptrs:          # 'T* const*': the const after a star qualifies the pointer before it, i.e. the next star's pointee
        raise AssertionError(ctype)
    return "".join(reversed(ptrs)) + base


def header_functions():
    text = re.sub(r"#[^\n]*", "", _strip_c(open(HEADER).read()))
    out = {}
    for m in re.finditer(r"(?:^|\n)\s*((?:const\s+)?[A-Za-z_][A-Za-z0-9_]*\s*\**)\s*(ughip_[a-z0-9_]+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        ret, name, args = " ".join(m.group(1).split()), m.group(2), " ".join(m.group(3).split())
        arg_types = []
        if args not in ("", "void"):
            for a in args.split(","):
                a = a.strip()
                t = re.match(r"(.*?)([A-Za-z_][A-Za-z0-9_]*)$", a)
                arg_types.append(c_type_to_rust(t.group(1).strip()))
        out[name] = (c_type_to_rust(ret) if ret != "void" else None, arg_types)
    return out


def rust_functions():
    text = re.sub(r"//[^\n]*", "", open(FFI).read())
    block = re.search(r'extern "C" \{(.*?)\n\}', text, flags=re.S).group(1)
    out = {}
    for m in re.finditer(r"pub fn (ughip_[a-z0-9_]+)\s*\((.*?)\)\s*(?:->\s*([^;]+?))?\s*;", block, flags=re.S):
        name, args, ret = m.group(1), " ".join(m.group(2).split()), m.group(3)
        arg_types = [a.split(":", 1)[1].strip() for a in args.split(",") if a.strip()]
        out[name] = (" ".join(ret.split()) if ret else None, arg_types)
    return out


def test_every_header_function_is_declared_in_ffi_rs_with_the_same_signature():
    c, r = header_functions(), rust_functions()
    assert len(c) >= 50, "the header parser lost declarations"
    assert sorted(c) == sorted(r), f"only in the header: {sorted(set(c) - set(r))}; only in ffi.rs: {sorted(set(r) - set(c))}"
    for name in c:
        assert c[name][0] == r[name][0], f"{name}: return type {c[name][0]} in the header, {r[name][0]} in ffi.rs"
        assert c[name][1] == r[name][1], f"{name}: arguments {c[name][1]} in the header, {r[name][1]} in ffi.rs"


def header_structs():
    text = _strip_c(open(HEADER).read())
    out = {}
    for m in re.finditer(r"typedef struct (ughip_[a-z_]+) \{(.*?)\} \1;", text, flags=re.S):
        fields = []
        for line in m.group(2).split(";"):
            line = " ".join(line.split())
            if not line:
                continue
            t = re.match(r"(.*?)([A-Za-z_][A-Za-z0-9_]*)$", line)
            fields.append((t.group(2), c_type_to_rust(t.group(1).strip())))
        out[C_TO_RUST_BASE[m.group(1)]] = fields
    return out


def rust_structs():
    text = re.sub(r"//[^\n]*", "", open(FFI).read())
    out = {}
    for m in re.finditer(r"#\[repr\(C\)\]\s*(?:#\[[^\]]*\]\s*)*pub struct (\w+) \{(.*?)\}", text, flags=re.S):
        fields = []
        for f in m.group(2).split(","):
            f = " ".join(f.split())
            if f:
                name, ty = f.replace("pub ", "").split(":", 1)
                fields.append((name.strip(), ty.strip()))
        out[m.group(1)] = fields
    return out


def test_repr_c_structs_match_the_header_field_for_field():
    c, r = header_structs(), rust_structs()
    assert set(c) == {"UghipA", "UghipInstr", "UghipKernelArg", "UghipSsa", "UghipFuncInfo"}
    assert set(c) == set(r)
    for name in c:
        assert c[name] == r[name], f"{name}: {c[name]} in the header, {r[name]} in ffi.rs"


def test_dtype_codes_and_constants_match():
    text = _strip_c(open(HEADER).read())
    rust = open(FFI).read()
    for name in ("BF16", "F16", "F32", "I32", "I64"):
        c_val = int(re.search(rf"UGHIP_{name}\s*=\s*(\d+)", text).group(1))
        r_val = int(re.search(rf"pub const UGHIP_{name}: c_int = (\d+);", rust).group(1))
        assert c_val == r_val, name
    c_shift = re.search(r"#define UGHIP_MATMUL_NOALLOC_SCRATCH_BYTES \((\d+)u << (\d+)\)", open(HEADER).read())
    r_shift = re.search(r"pub const UGHIP_MATMUL_NOALLOC_SCRATCH_BYTES: usize = (\d+) << (\d+);", rust)
    assert c_shift.groups() == r_shift.groups()


def test_instruction_codes_used_by_the_serialiser_match_the_header():
    """runtime.rs writes `op: N` literals in the declaration order of ssa::Instr; the header's UGHIP_I_* say which N
    means what."""
    text = _strip_c(open(HEADER).read())
    codes = {m.group(1): int(m.group(2)) for m in re.finditer(r"UGHIP_I_([A-Z_]+)\s*=\s*(\d+)", text)}
    runtime = open(os.path.join(RUST, "ug-hip", "src", "runtime.rs")).read()
    want = {"DefineAcc": "DEFINE_ACC", "DefineGlobal": "DEFINE_GLOBAL", "DefineLocal": "DEFINE_LOCAL", "Special": "SPECIAL", "Const": "CONST", "Unary": "UNARY",
            "Binary": "BINARY", "Range": "RANGE", "Load": "LOAD", "Assign": "ASSIGN", "EndRange": "END_RANGE", "If": "IF", "EndIf": "END_IF", "Store": "STORE",
            "Barrier": "BARRIER", "ReduceLocal": "REDUCE_LOCAL"}
    body = runtime[runtime.index("fn wire_instr"):runtime.index("/// The POD image of a kernel")]
    for variant, cname in want.items():
        m = re.search(rf"\n\s+{variant}\b[^=]*=>\s*(?:\{{.*?)?UghipInstr \{{ op: (\d+)", body, flags=re.S)
        assert m, variant
        assert int(m.group(1)) == codes[cname], f"{variant}: op {m.group(1)} in runtime.rs, UGHIP_I_{cname} = {codes[cname]}"


def test_every_entry_point_the_rust_files_call_exists():
    declared = set(rust_functions())
    for path in (os.path.join(RUST, "ug-hip", "src", "runtime.rs"), os.path.join(RUST, "ug-llama", "src", "hip_ops.rs")):
        used = set(re.findall(r"ffi::(ughip_[a-z0-9_]+)", open(path).read()))
        assert used, path
        assert used <= declared, f"{path} calls undeclared {sorted(used - declared)}"
    ops = open(os.path.join(RUST, "ug-llama", "src", "hip_ops.rs")).read()
    for op in ("rope_i", "rope", "cat", "custom_softmax", "causal_mask"):      # ug-llama/src/main.rs:22-28
        assert re.search(rf"fn {op}\(", ops), op
